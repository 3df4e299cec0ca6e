#!/usr/bin/env python3
"""Benchmark of the weight-only quantized matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --mode sweep --sweep decode8b|prefill8b|llama70b|w4a8|moe   (tables of the other
                                                   benchmark configurations, one JSON line per case)

Workload (the configuration the headline metric is quoted on): W4A16, group 128, bf16
activations/scales/zeros, M = 1 — the four linear layers of one Llama-3-8B decoder layer
(qkv K=4096 N=6144, o K=4096 N=4096, gate_up K=4096 N=28672, down K=14336 N=4096).  One "step" is
one pass over those four matmuls.  Steps rotate over several distinct copies of the weights
(more than the 256 MB last-level cache), so weights always come from HBM.  The timed K steps are
captured in one HIP graph and replayed, so launches are back to back with no Python in between.

`value` = algorithmic bytes of a step / time of a step (inputs resident in HBM).  `roofline`
describes the dominant kernel (the gate_up GEMV), timed on its own with HIP events on the launch
stream.  `cpu_baseline` times the reference's CPU path (torch dequantize + float32 matmul) on the
host cores for the same step.  `gemm` (extra field) reports the prefill regime at M = 4096.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import torch

from __graft_entry__ import import_package

METRIC = "W4A16 g128 GEMM: HBM GB/s at M=1, TFLOP/s at M=4096 (Llama-3-8B shapes)"
SHAPES_8B = [("qkv", 4096, 6144), ("o_proj", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]
SHAPES_70B = [("qkv", 8192, 10240), ("o_proj", 8192, 8192), ("gate_up", 8192, 57344), ("down", 28672, 8192)]
GROUP = 128
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_FP8_PEAK_TFLOPS = 5000.0
CACHE_BYTES = 256 << 20  # last-level (Infinity) cache; rotation must exceed it
TRAFFIC_PROFILE = "profiles/stream_gemv_gate_up_m1_hbm_traffic.md"


def recorded_traffic_bytes(launched):
    """HBM bytes per launch of the dominant kernel as the tracked rocprofv3 --pmc summary records them
    (FETCH_SIZE / WRITE_SIZE runs calibrated with a 256 MiB copy; the line `traffic_bytes_per_launch: N`
    of TRAFFIC_PROFILE).  Counters cannot be read from inside this process; None when the summary is
    missing or was taken on another kernel or launch shape than `launched`, which is what the library
    reports (woq_last_launch) for the launch this run timed (the summary's line `launch: ...`)."""
    import os
    import re
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), TRAFFIC_PROFILE)
    try:
        text = open(path).read()
    except OSError:
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    k = re.search(r"^launch:\s*(.+?)\s*$", text, re.M)
    if not m or not k or k.group(1) != launched:
        return None
    return int(m.group(1))


def last_launch(pkg):
    """What the library launched for this thread's last matmul call (kernel family and launch shape)."""
    return (pkg._lib.lib.woq_last_launch() or b"").decode()


def algorithmic_bytes(m, k, n, bits=4, group=GROUP, n_sz=2, act_bytes=2):
    """Every operand once: packed weights + scales(+zeros) + activations + output."""
    sz = (k // group) * n * 2 * n_sz if group else n * 2
    return k * n * bits // 8 + sz + m * k * act_bytes + m * n * 2


def make_layer(pkg, dev, k, n, seed, group=GROUP):
    """Synthetic tensors of the benchmark configuration: W ~ N(0, 0.02) quantized to uint4 with
    group 128 (or 64) along K (asymmetric min/max), bf16 scales, bf16 zeros = (8 - zp) * scale."""
    g = torch.Generator(device=dev).manual_seed(seed)
    w = torch.randn((k, n), generator=g, device=dev, dtype=torch.float32) * 0.02
    wg = w.view(k // group, group, n)
    mx, mn = wg.amax(1), wg.amin(1)
    scale = ((mx - mn).clamp_min(1e-8) / 15.0).to(torch.bfloat16)
    sf = scale.float()
    zp = torch.round(-mn / sf).clamp(0, 15)
    qu = (torch.round(wg / sf[:, None, :]) + zp[:, None, :]).clamp(0, 15)
    q = (qu - 8).to(torch.int8).view(k, n)
    zeros = ((8.0 - zp) * sf).to(torch.bfloat16)
    packed = ((q[:, 0::2] & 0xF) | (q[:, 1::2] << 4)).to(torch.int8).cpu().contiguous()
    wq = pkg.ops.preprocess_weights_for_mixed_gemm(packed, torch.quint4x2, torch.bfloat16).to(dev)
    return dict(k=k, n=n, q=q, weight=wq, scales=scale.contiguous(), zeros=zeros.contiguous(), group=group,
                algo=pkg.functional.ZERO)


def make_layer_int8(pkg, dev, k, n, seed):
    """W8A16 per-channel: W ~ N(0, 0.02) quantized symmetrically to int8, one bf16 scale per column."""
    g = torch.Generator(device=dev).manual_seed(seed)
    w = torch.randn((k, n), generator=g, device=dev, dtype=torch.float32) * 0.02
    scale = (w.abs().amax(0) / 127.0).to(torch.bfloat16)
    q = torch.round(w / scale.float()).clamp(-128, 127).to(torch.int8)
    wq = pkg.ops.preprocess_weights_for_mixed_gemm(q.cpu().contiguous(), torch.int8, torch.bfloat16).to(dev)
    return dict(k=k, n=n, q=q, weight=wq, scales=scale.contiguous(), zeros=None, group=0,
                algo=pkg.functional.INT8_WEIGHT)


def copies_beyond_cache(weight_bytes, factor=2):
    return max(2, -(-factor * CACHE_BYTES // weight_bytes))


def rotated_copies(layer, copies):
    """Distinct device buffers holding the same tiles in rolled order: different addresses for
    the caches, still valid weights (any byte pattern is)."""
    out = [layer]
    tiles = layer["weight"].view(-1, 1024)
    for r in range(1, copies):
        c = dict(layer)
        c["weight"] = tiles.roll(977 * r + 1, 0).contiguous().view_as(layer["weight"])
        c["scales"] = layer["scales"].roll(r, 0).contiguous()
        if layer["zeros"] is not None:
            c["zeros"] = layer["zeros"].roll(r, 0).contiguous()
        out.append(c)
    return out


_workspaces = {}


def workspace_for(pkg, m, layer, dev):
    """One scratch buffer per (m, n, k, kind), sized by woq_workspace_bytes and reused by every launch
    (the caller of the library owns the workspace; nothing is allocated inside the timed region)."""
    key = (m, layer["n"], layer["k"], layer["algo"])
    if key not in _workspaces:
        need = pkg._lib.lib.woq_workspace_bytes(m, layer["n"], layer["k"], layer["algo"], pkg._lib.BF16)
        _workspaces[key] = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
    return _workspaces[key]


def launch(pkg, act, layer, out, regime=0):
    F = pkg.functional
    F.woq_matmul_raw(act, None, layer["weight"], layer["scales"], layer["zeros"], None, n=layer["n"], k=layer["k"],
                     group_size=layer["group"], quant_algo=layer["algo"], out_dtype=torch.bfloat16, out=out,
                     regime=regime, workspace=workspace_for(pkg, act.shape[0], layer, act.device))


SETTLE_S = 0.08  # untimed replays before a timed one; see time_graph


def time_graph(fn_body, launches, repeats=1, settle_s=SETTLE_S, first=None):
    """Captures fn_body() (which issues `launches` kernels) in a HIP graph, replays it untimed until
    `settle_s` seconds have passed, then times one replay with HIP events on the replay stream and with
    the host clock (`repeats` > 1: the median of that many timed replays).

    Why the untimed replays: when load starts on an idle GPU, the first millisecond runs at full clocks,
    then the power management pulls the clocks down (kernels take up to 1.5x as long) and lets them come
    back over the next 20-40 ms, after which the time per launch stays flat for seconds.  A timed replay
    without the settling phase lands somewhere on that curve.  `first`, a dict, receives the event time
    of the very first replay ("first_replay_s"), the figure a measurement without settling would give."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    timed = []
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            fn_body()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        if first is not None:
            first["first_replay_s"] = e0.elapsed_time(e1) * 1e-3
        t_settle = time.perf_counter()
        while time.perf_counter() - t_settle < settle_s:
            graph.replay()
            graph.replay()
            torch.cuda.synchronize()
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            timed.append(((t1 - t0), e0.elapsed_time(e1) * 1e-3, launches))
    timed.sort(key=lambda t: t[1])
    return timed[len(timed) // 2]


def bench_decode(pkg, dev, steps, warmup, m=1):
    per_step_bytes = sum(algorithmic_bytes(m, k, n) for _, k, n in SHAPES_8B)
    weight_bytes = sum(k * n // 2 for _, k, n in SHAPES_8B)
    copies = copies_beyond_cache(weight_bytes, 3)  # the step's own rotation: >= 3x the cache
    # each shape is also timed alone, so each gets enough copies to exceed the cache by itself
    layers = [rotated_copies(make_layer(pkg, dev, k, n, 2000 + i), max(copies, copies_beyond_cache(k * n // 2)))
              for i, (_, k, n) in enumerate(SHAPES_8B)]
    g = torch.Generator(device=dev).manual_seed(2999)
    acts = {k: torch.randn((m, k), generator=g, device=dev).to(torch.bfloat16) for k in (4096, 14336)}
    outs = [torch.empty((m, n), dtype=torch.bfloat16, device=dev) for _, _, n in SHAPES_8B]

    def step(s):
        for i, (_, k, _) in enumerate(SHAPES_8B):
            launch(pkg, acts[k], layers[i][s % len(layers[i])], outs[i])

    for s in range(warmup):
        step(s)
    torch.cuda.synchronize()
    first = {}
    host_s, ev_s, _ = time_graph(lambda: [step(s) for s in range(steps)], steps * len(SHAPES_8B), first=first)

    # dominant kernel on its own: the gate_up GEMV
    gi = 2
    _, gk, gn = SHAPES_8B[gi]
    # (a graph launch costs about 40 us before its first kernel starts, whatever its length: 400 launches per
    # replay keep that below 1 % of a launch; the step's own timing above is exactly `steps` steps, as asked)
    reps = max(steps, 400)
    _, dom_s, dom_launches = time_graph(
        lambda: [launch(pkg, acts[gk], layers[gi][r % len(layers[gi])], outs[gi]) for r in range(reps)], reps)
    dom_launch = last_launch(pkg)  # the kernel and launch shape the timed launches ran on
    dom_bytes = algorithmic_bytes(m, gk, gn)
    dom_dur = dom_s / dom_launches
    per_shape = {}
    for i, (name, k, n) in enumerate(SHAPES_8B):
        _, s_s, s_l = time_graph(
            lambda: [launch(pkg, acts[k], layers[i][r % len(layers[i])], outs[i]) for r in range(reps)], reps)
        per_shape[name] = dict(us=round(s_s / s_l * 1e6, 3), gbs=round(algorithmic_bytes(m, k, n) / (s_s / s_l) / 1e9, 1))
    return dict(host_s=host_s, ev_s=ev_s, first_replay_s=first["first_replay_s"], per_step_bytes=per_step_bytes, copies=copies, dom_dur=dom_dur,
                dom_bytes=dom_bytes, dom_launch=dom_launch, per_shape=per_shape, layers=layers, acts=acts)


def bench_cpu_baseline(layers, acts, m=1, budget_s=15.0):
    """The reference's CPU path (tensorrt_llm/quantization/functional.py:269-290 semantics) on the host
    cores, two timings: (i) dequantize with torch, then a float32 matmul - `value`; (ii) the float32
    matmul alone on weights dequantized beforehand - `matmul_only`.  Both in the metric's unit, i.e.
    the step's algorithmic bytes (of the QUANTIZED operands) per second."""
    from __graft_entry__ import import_oracle
    o = import_oracle()
    host = []
    for i, (_, k, n) in enumerate(SHAPES_8B):
        l = layers[i][0]
        host.append((acts[k].float().cpu(), l["q"].cpu(), l["scales"].float().cpu(), l["zeros"].float().cpu()))
    per_step_bytes = sum(algorithmic_bytes(m, k, n) for _, k, n in SHAPES_8B)

    def median_time(fn, budget, most):
        times = []
        t_start = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_start < budget and len(times) < most):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2], len(times)

    med, passes = median_time(lambda: [o.torch_cpu_dequant_matmul(a, q, s, z, GROUP) for a, q, s, z in host],
                              budget_s, 20)
    # (ii): weights dequantized once, outside the timed region
    dense = []
    for a, q, s, z in host:
        w = q.to(torch.float32) * s.repeat_interleave(GROUP, dim=0) + z.repeat_interleave(GROUP, dim=0)
        dense.append((a, w))
    med_mm, passes_mm = median_time(lambda: [a @ w for a, w in dense], budget_s / 3, 40)
    return dict(value=round(per_step_bytes / med / 1e9, 3), unit="GB/s", cores=torch.get_num_threads(), kind="port",
                matmul_only=round(per_step_bytes / med_mm / 1e9, 3),
                sample="%d passes over the same 4-matmul step (torch dequant + fp32 matmul), median %.1f ms; "
                       "%d passes of the fp32 matmuls alone on pre-dequantized weights, median %.1f ms"
                       % (passes, med * 1e3, passes_mm, med_mm * 1e3))


def bench_gemm(pkg, dev, m=4096, reps=40):
    """Prefill regime, largest shape (gate_up): TFLOP/s at M = 4096, as the average of `reps` launches
    back to back (a replay of ~30 ms, after the settling replays every timing here has)."""
    try:
        name, k, n = SHAPES_8B[2]
        layer = make_layer(pkg, dev, k, n, 3000)
        g = torch.Generator(device=dev).manual_seed(3999)
        act = torch.randn((m, k), generator=g, device=dev).to(torch.bfloat16)
        out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        launch(pkg, act, layer, out)
        torch.cuda.synchronize()
        # the launches replay from a HIP graph; the median of three timed replays
        _, sec, launches = time_graph(lambda: [launch(pkg, act, layer, out) for _ in range(reps)], reps, repeats=3)
        launched = last_launch(pkg)
        sec /= launches
        tf = 2.0 * m * n * k / sec / 1e12
        # context, not a baseline: the vendor library's plain bf16 x bf16 GEMM (no dequantize) of the
        # same shape on this box, through torch.matmul
        dense = torch.randn((k, n), generator=g, device=dev).to(torch.bfloat16)
        torch.matmul(act, dense, out=out)
        torch.cuda.synchronize()
        _, lib_sec, _ = time_graph(lambda: [torch.matmul(act, dense, out=out) for _ in range(reps)], reps, repeats=3)
        lib_tf = 2.0 * m * n * k / (lib_sec / reps) / 1e12
        return dict(shape=name, m=m, us=round(sec * 1e6, 1), tflops=round(tf, 1),
                    frac_of_bf16_peak=round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                    library_dense_bf16_gemm_tflops=round(lib_tf, 1),
                    # the M = 4096 half of the metric in the shape of `roofline`
                    roofline={"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                              "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                              "kernel": "%s (bf16 x int4 g128 + zeros) on gate_up K=%d N=%d M=%d" % (launched, k, n, m),
                              "flop_per_launch": 2.0 * m * n * k, "us_per_launch": round(sec * 1e6, 1)})
    except Exception as e:  # the decode line is still valid without the prefill extra
        return dict(error=str(e)[:200])


def w4a8_setup(pkg, dev, m, k, n, seed=4000, copies=1, layers=None):
    """W4A8 operands of the benchmark's kind: int4 symmetric g128 weights (same gfx950 layout),
    fp16 group scales, activations already smoothed and cast to e4m3, alpha in the epilogue.
    run(r) uses weight copy r % copies."""
    F = pkg.functional
    layers = layers or rotated_copies(make_layer(pkg, dev, k, n, seed), copies)
    scales = [l["scales"].to(torch.float16) for l in layers]
    g = torch.Generator(device=dev).manual_seed(seed + 1)
    act = (torch.randn((m, k), generator=g, device=dev) * 0.5).to(torch.float8_e4m3fn)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)

    def run(r=0):
        c = r % copies
        F.woq_matmul_raw(act, None, layers[c]["weight"], scales[c], None, None, n=n, k=k, group_size=GROUP,
                         quant_algo=F.FP8_ALPHA, alpha=0.5, out_dtype=torch.bfloat16, out=out)
    return run


def bench_w4a8(pkg, dev, m=4096, reps=40):
    """W4A8 (fp8 MFMA) on gate_up: TFLOP/s at M = 4096 against the 5 PFLOP/s dense fp8 peak."""
    try:
        name, k, n = SHAPES_8B[2]
        run = w4a8_setup(pkg, dev, m, k, n)
        run()
        torch.cuda.synchronize()
        _, sec, launches = time_graph(lambda: [run() for _ in range(reps)], reps, repeats=3)
        sec /= launches
        tf = 2.0 * m * n * k / sec / 1e12
        return dict(shape=name, m=m, us=round(sec * 1e6, 1), tflops=round(tf, 1),
                    frac_of_fp8_peak=round(tf / MFMA_FP8_PEAK_TFLOPS, 4))
    except Exception as e:
        return dict(error=str(e)[:200])


def run_for_counters(pkg, dev, mode, reps=20, shape=None, replay_ms=0):
    """Helpers for `rocprofv3` runs (one counter set per --pmc run): `dominant` launches only the
    dominant kernel (gate_up GEMV, rotating weight copies); `gemm<M>` launches the GEMM regime on
    gate_up at M rows (256-row tiles at 4096, 64-row tiles at 128); `copy` runs a plain device-to-device
    copy of a known size (256 MiB read + 256 MiB written per launch), whose FETCH_SIZE /
    WRITE_SIZE readings calibrate the counters.  Each mode issues `reps` plain launches; with
    `replay_ms` it then replays 40 launches from a HIP graph for that long and times three more
    replays, as the sweeps do - for kernel traces (see summarize_trace), not for counter runs."""
    def finish(issue, line):
        for r in range(reps):
            issue(r)
        torch.cuda.synchronize()
        line["launches"] = reps
        if replay_ms > 0:
            first = {}
            _, sec, launches = time_graph(lambda: [issue(r) for r in range(40)], 40, repeats=3,
                                          settle_s=replay_ms * 1e-3, first=first)
            line["replayed"] = {"ms": replay_ms, "launches_per_replay": 40,
                                "us_per_launch": round(sec / launches * 1e6, 2),
                                "first_replay_us_per_launch": round(first["first_replay_s"] / 40 * 1e6, 2)}
        print(json.dumps(line))

    if mode == "copy":
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        finish(lambda r: dst.copy_(src),
               {"mode": "copy", "bytes_read_per_launch": 256 << 20, "bytes_written_per_launch": 256 << 20})
        return
    if mode == "w4a8_decode":
        _, k, n = SHAPES_70B[2]
        copies = copies_beyond_cache(k * n // 2)
        run = w4a8_setup(pkg, dev, 1, k, n, copies=copies)
        run(0)
        finish(run, {"mode": mode, "kernel": last_launch(pkg) + " on 70B gate_up K=8192 N=57344 M=1",
                     "algorithmic_bytes_per_launch": algorithmic_bytes(1, k, n, 4, GROUP, 1, 1)})
        return
    if mode == "moe_decode":
        F = pkg.functional
        experts, k, n = 8, 4096, 28672
        layers = [make_layer(pkg, dev, k, n, 6000 + e) for e in range(experts)]
        copies = copies_beyond_cache(experts * k * n // 2)
        weight = [torch.stack([l["weight"] for l in layers]).roll(r, 0).contiguous() for r in range(copies)]
        scales = torch.stack([l["scales"] for l in layers]).contiguous()
        zeros = torch.stack([l["zeros"] for l in layers]).contiguous()
        rows = torch.tensor([5, 1, 4, 4, 6, 3, 8, 1])
        total = torch.cumsum(rows, 0).to(torch.int64).to(dev)
        act = torch.randn((int(rows.sum()), k), device=dev).to(torch.bfloat16)
        out = torch.empty((act.shape[0], n // 2), dtype=torch.bfloat16, device=dev)
        by = experts * (k * n // 2 + (k // GROUP) * n * 4) + act.numel() * 2 + out.numel() * 2
        finish(lambda r: F.woq_grouped_matmul_raw(act, weight[r % copies], scales, zeros, None, total, n=n, k=k,
                                                  group_size=GROUP, quant_algo=F.ZERO, activation="swiglu", out=out),
               {"mode": mode, "kernel": "grouped streaming kernel, 8 experts K=4096 N=28672 + swiglu, "
                                        "32 rows (16 tokens, top-2)", "algorithmic_bytes_per_launch": by})
        return
    _, k, n = SHAPES_8B[2]
    shapes = dict([("8b_" + nm, (kk, nn)) for nm, kk, nn in SHAPES_8B] + [("70b_" + nm, (kk, nn)) for nm, kk, nn in SHAPES_70B])
    if mode.startswith("w4a8_") and mode[5:].isdigit():
        m = int(mode[5:])
        if shape:
            k, n = shapes[shape]
        copies = copies_beyond_cache(k * n // 2) if m <= 256 else 1
        run = w4a8_setup(pkg, dev, m, k, n, copies=copies)
        run(0)
        finish(run, {"mode": mode, "kernel": "%s on %s K=%d N=%d M=%d" % (last_launch(pkg), shape or "gate_up", k, n, m),
                     "flop_per_launch": 2.0 * m * n * k})
        return
    if mode.startswith("gemm"):
        m = int(mode[4:] or 4096)
        if shape:  # another layer shape than the 8B gate_up: "70b_qkv", "8b_down", ...
            k, n = shapes[shape]
        # weights rotate over copies beyond the last-level cache while they matter (M <= 256), as in the sweeps
        copies = min(copies_beyond_cache(k * n // 2), 64) if m <= 256 else 1
        layers = rotated_copies(make_layer(pkg, dev, k, n, 2002), copies)
        act = torch.randn((m, k), device=dev).to(torch.bfloat16)
        out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        launch(pkg, act, layers[0], out)
        finish(lambda r: launch(pkg, act, layers[r % copies], out),
               {"mode": mode, "kernel": "%s on %s K=%d N=%d M=%d" % (last_launch(pkg), shape or "8b_gate_up", k, n, m),
                "flop_per_launch": 2.0 * m * n * k, "algorithmic_bytes_per_launch": algorithmic_bytes(m, k, n)})
        return
    if mode == "dominant70b":  # the same GEMV on the Llama-3-70B gate_up
        _, k, n = SHAPES_70B[2]
    copies = max(2, -(-3 * CACHE_BYTES // (k * n // 2)))
    layers = rotated_copies(make_layer(pkg, dev, k, n, 2002), copies)
    act = torch.randn((1, k), device=dev).to(torch.bfloat16)
    out = torch.empty((1, n), dtype=torch.bfloat16, device=dev)
    launch(pkg, act, layers[0], out)
    finish(lambda r: launch(pkg, act, layers[r % copies], out),
           {"mode": mode, "kernel": last_launch(pkg) + " on gate_up K=%d N=%d M=1" % (k, n),
            "algorithmic_bytes_per_launch": algorithmic_bytes(1, k, n)})


def summarize_trace(path):
    """Reads a `rocprofv3 --kernel-trace --output-format csv` kernel trace and prints, per kernel, the
    dispatch count and the durations (end - begin stamp, us): mean of all, median of the first 20
    dispatches (a GPU that was idle just before), largest median over any 40 consecutive dispatches (the dip
    of the clocks that follows), median of the last quarter (settled).  No GPU needed."""
    import csv
    import statistics as st
    by_kernel = {}
    for row in csv.DictReader(open(path)):
        by_kernel.setdefault(row["Kernel_Name"], []).append((int(row["Start_Timestamp"]), int(row["End_Timestamp"])))
    for name, stamps in sorted(by_kernel.items(), key=lambda kv: -sum(e - b for b, e in kv[1])):
        stamps.sort()
        d = [(e - b) / 1e3 for b, e in stamps]
        worst = max(st.median(d[i:i + 40]) for i in range(0, max(1, len(d) - 39), 20))
        print(json.dumps({"kernel": name[:120], "dispatches": len(d), "mean_us": round(st.mean(d), 2),
                          "first20_median_us": round(st.median(d[:20]), 2), "worst40_median_us": round(worst, 2),
                          "last_quarter_median_us": round(st.median(d[-max(1, len(d) // 4):]), 2)}))


SWEEPS = {
    # name: (shapes, kinds, row counts); kind = ("w4a16", group) | ("w8a16", 0) | ("w4a8", 128)
    "decode8b": (SHAPES_8B, [("w4a16", 128)], [1, 4, 8, 16]),
    "prefill8b": (SHAPES_8B, [("w4a16", 128), ("w8a16", 0)], [512, 2048, 4096, 8192]),
    "llama70b": (SHAPES_70B, [("w4a16", 128), ("w4a16", 64)], [1, 2, 4, 8, 16, 32, 64, 128, 256]),
    "w4a8": (SHAPES_70B, [("w4a8", 128)], [1, 16, 256, 4096]),
}


def run_sweep(pkg, dev, which, tuned=False):
    """The benchmark's other configurations: one JSON line per (kind, shape, M) with the launch time,
    algorithmic GB/s and TFLOP/s.  Launches rotate over weight copies exceeding the last-level cache
    while M <= 256 (weight traffic matters there); all launches of a case replay from one HIP graph.
    With `tuned`, each layer is then profiled (woq_profile_tactics over the sweep's row counts) and
    timed again, and the line also carries the tuned tactic and its time."""
    F = pkg.functional
    shapes, kinds, ms = SWEEPS[which]
    for kind, group in kinds:
        for name, k, n in shapes:
            bits = 8 if kind == "w8a16" else 4
            copies = min(copies_beyond_cache(k * n * bits // 8), 64) if min(ms) <= 256 else 1
            if kind == "w8a16":
                layers = rotated_copies(make_layer_int8(pkg, dev, k, n, 5000), copies)
            else:
                layers = rotated_copies(make_layer(pkg, dev, k, n, 5000, group), copies)

            def time_case(m):
                reps = 40 if m <= 256 else 20
                if kind == "w4a8":
                    runner = w4a8_setup(pkg, dev, m, k, n, 5000, copies, layers)
                    body = lambda: [runner(r) for r in range(reps)]
                    runner(0)
                else:
                    act = torch.randn((m, k), device=dev).to(torch.bfloat16)
                    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
                    body = lambda: [launch(pkg, act, layers[r % copies], out) for r in range(reps)]
                    launch(pkg, act, layers[0], out)
                torch.cuda.synchronize()
                _, sec, launches = time_graph(body, reps, repeats=3)
                return sec / launches * 1e6

            F.clear_tactics()
            base = {m: time_case(m) for m in ms}
            best, tactic = {}, {}
            if tuned and kind != "w4a8":
                lay = layers[0]
                F.profile_tactics(None, lay["weight"], lay["scales"], lay["zeros"], None, n=n, k=k, group_size=group,
                                  quant_algo=lay["algo"], dtype=torch.bfloat16, min_m=min(ms), max_m=max(ms))
                for m in ms:
                    tactic[m] = F.describe_tactic(m, n, k, group, lay["algo"], torch.bfloat16)
                    best[m] = time_case(m)
                F.clear_tactics()
            for m in ms:
                us = base[m]
                n_sz = 1 if kind != "w4a16" else 2  # scales only, or scales + zeros
                by = algorithmic_bytes(m, k, n, bits, group, n_sz, 1 if kind == "w4a8" else 2)
                line = {"sweep": which, "kind": kind, "group": group, "shape": name, "k": k, "n": n, "m": m,
                        "us": round(us, 2), "gbs": round(by / us / 1e3, 1),
                        "tflops": round(2.0 * m * n * k / us / 1e6, 1), "weight_copies": copies}
                if m in best:
                    line.update({"tuned_us": round(best[m], 2), "tuned": tactic[m]})
                print(json.dumps(line), flush=True)
            layers = None
            torch.cuda.empty_cache()


def run_moe_sweep(pkg, dev):
    """Grouped (mixture-of-experts) matmul on Mixtral-8x7B expert shapes: 8 experts, W4A16 g128 with
    bf16 scales + zeros, top-2 routing of T tokens drawn uniformly (seeded), rows sorted by expert.
    One JSON line per (shape, T): launch time, algorithmic GB/s (weights of the experts that own
    rows + scales + activations + outputs) and TFLOP/s."""
    F = pkg.functional
    experts, top_k = 8, 2
    for name, k, n, activation in [("fc1 gate_up", 4096, 28672, "identity"), ("fc1 gate_up + swiglu", 4096, 28672, "swiglu"),
                                   ("fc2 down", 14336, 4096, "identity")]:
        layers = [make_layer(pkg, dev, k, n, 6000 + e) for e in range(experts)]
        copies = copies_beyond_cache(experts * k * n // 2)
        weight = [torch.stack([l["weight"] for l in layers]).roll(r, 0).contiguous() for r in range(copies)]
        scales = torch.stack([l["scales"] for l in layers]).contiguous()
        zeros = torch.stack([l["zeros"] for l in layers]).contiguous()
        layers = None
        for tokens in [1, 4, 16, 64, 256, 1024, 4096]:
            g = torch.Generator().manual_seed(tokens)
            picks = torch.stack([torch.randperm(experts, generator=g)[:top_k] for _ in range(tokens)]).flatten()
            rows = torch.bincount(picks, minlength=experts)
            total = torch.cumsum(rows, 0).to(torch.int64).to(dev)
            m = int(rows.sum())
            act = torch.randn((m, k), device=dev).to(torch.bfloat16)
            n_out = n // 2 if activation == "swiglu" else n
            out = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
            reps = 20 if m <= 512 else 4

            def run(r):
                F.woq_grouped_matmul_raw(act, weight[r % copies], scales, zeros, None, total, n=n, k=k,
                                         group_size=GROUP, quant_algo=F.ZERO, activation=activation, out=out)
            run(0)
            torch.cuda.synchronize()
            _, sec, launches = time_graph(lambda: [run(r) for r in range(reps)], reps, repeats=3)
            us = sec / launches * 1e6
            active = int((rows > 0).sum())
            by = active * (k * n // 2 + (k // GROUP) * n * 4) + m * k * 2 + m * n_out * 2
            print(json.dumps({"sweep": "moe", "shape": name, "k": k, "n": n, "experts": experts, "tokens": tokens,
                              "rows": m, "rows_per_expert": rows.tolist(), "us": round(us, 2),
                              "gbs": round(by / us / 1e3, 1), "tflops": round(2.0 * m * n * k / us / 1e6, 1)}),
                  flush=True)
        weight = scales = zeros = None
        torch.cuda.empty_cache()


def run_ceilings(pkg, dev):
    """What the hardware allows, with this file's own timing (HIP graph replays, buffers rotating through
    1 GiB so that nothing is served from the last-level cache): plain streaming reads at the byte counts
    of the benchmark's GEMVs, an empty launch, and matrix-instruction-only kernels.  One JSON line."""
    import ctypes
    lib = pkg._lib.lib
    stream_of = lambda: ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    pool = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
    sink = torch.zeros(4096, dtype=torch.uint8, device=dev)
    out = {"mode": "ceilings", "reads": [], "hbm_peak_gbs": HBM_PEAK_GBS}
    # algorithmic bytes of the M = 1 GEMVs: 8B o_proj, qkv, down, gate_up, 70B gate_up (rounded to 64 KiB)
    for label, nbytes in [("8b_o_proj 8.9 MB", 8929280), ("8b_qkv 13.4 MB", 13389824), ("8b_down 31.2 MB", 31232000),
                          ("8b_gate_up 62.5 MB", 62455808), ("70b_gate_up 250 MB", 250478592)]:
        nbytes = nbytes // 65536 * 65536
        copies = (1 << 30) // nbytes
        entry = {"like": label, "bytes": nbytes}
        for nt in (0, 1):  # ordinary loads / loads with the non-temporal hint (the streaming kernels' weight loads)
            best = None
            for kib, u in [(4, 4), (8, 8), (16, 8), (32, 4), (64, 8)]:
                def body(reps=40):
                    for r in range(reps):
                        pkg._lib.check(lib.woq_probe_read(ctypes.c_void_p(pool.data_ptr() + (r % copies) * nbytes),
                                                          ctypes.c_size_t(nbytes), kib, u, nt,
                                                          ctypes.c_void_p(sink.data_ptr()), stream_of()))
                body(3)
                torch.cuda.synchronize()
                _, sec, launches = time_graph(body, 40, repeats=3)
                us = sec / launches * 1e6
                if best is None or us < best[0]:
                    best = (us, kib, u)
            tag = "nontemporal_" if nt else ""
            entry.update({tag + "us": round(best[0], 2), tag + "gbs": round(nbytes / best[0] / 1e3, 1),
                          tag + "frac_of_peak": round(nbytes / best[0] / 1e3 / HBM_PEAK_GBS, 4),
                          tag + "kib_per_wave": best[1], tag + "loads_in_flight": best[2]})
        out["reads"].append(entry)

    def empty(reps=200):
        for _ in range(reps):
            pkg._lib.check(lib.woq_probe_empty(ctypes.c_void_p(sink.data_ptr()), stream_of()))
    empty(5)
    torch.cuda.synchronize()
    _, sec, launches = time_graph(empty, 200, repeats=3)
    out["empty_launch_us"] = round(sec / launches * 1e6, 3)
    for kind, name, peak in [(0, "v_mfma_f32_16x16x32_bf16", MFMA_BF16_PEAK_TFLOPS),
                             (2, "v_mfma_f32_32x32x16_bf16", MFMA_BF16_PEAK_TFLOPS),
                             (1, "v_mfma_f32_16x16x128_f8f6f4 (e4m3)", MFMA_FP8_PEAK_TFLOPS)]:
        for random_operands in (0, 1):
            flop = [0.0]

            def body(reps=8):
                for _ in range(reps):
                    flop[0] = lib.woq_probe_mfma(kind, random_operands, 20000, 256, ctypes.c_void_p(sink.data_ptr()),
                                                 stream_of())
            body(1)
            torch.cuda.synchronize()
            _, sec, launches = time_graph(body, 8, repeats=3)
            tf = flop[0] / (sec / launches) / 1e12
            entry = {"instruction": name, "operands": "random" if random_operands else "constant",
                     "tflops": round(tf, 1), "peak": peak, "frac_of_peak": round(tf / peak, 4),
                     "ms_per_launch": round(sec / launches * 1e3, 3)}
            if kind != 2:  # the 16x16 probes leave shader-clock cycles and 100 MHz ticks of one wavefront's loop
                counts = sink.view(torch.int32)[1020:1022].tolist()
                if counts[1] > 0:
                    entry["shader_clock_mhz"] = round((counts[0] & 0xFFFFFFFF) / counts[1] * 100.0)
            out.setdefault("mfma", []).append(entry)
    print(json.dumps(out))


def run_timeline(pkg, dev, shape):
    """Per-wavefront time stamps of the row decode kernel (M = 1, W4A16 g128) on one layer shape.  Needs the
    library built with `python tensorrt-llm_amd/build.py --timeline` and selected through
    WOQ_LIB_PATH=tensorrt-llm_amd/libwoq_timeline.so: its row kernel stamps the constant 100 MHz clock at seven
    points of every wavefront and stores them where WOQ_TRACE_PTR (read at launch) points.  Twelve launches
    replay from one graph after the usual settling; the stamps of launches 3-11 are reported as percentiles
    over the wavefronts, in us after the launch's first wavefront started, medians over the launches.  The
    stamps cost time (the same launch runs about a tenth slower than in the plain library): the figures
    show where a wavefront waits, not what the plain kernel takes."""
    import os
    import numpy as np
    k, n = dict([("8b_" + nm, (kk, nn)) for nm, kk, nn in SHAPES_8B]
                + [("70b_" + nm, (kk, nn)) for nm, kk, nn in SHAPES_70B])[shape or "8b_gate_up"]
    copies = copies_beyond_cache(k * n // 2, 3)
    layers = rotated_copies(make_layer(pkg, dev, k, n, 2002), copies)
    act = torch.randn((1, k), device=dev).to(torch.bfloat16)
    out = torch.empty((1, n), dtype=torch.bfloat16, device=dev)
    launches = 12
    waves_max = (n // 16) * 16  # one workgroup per strip, at most 16 wavefronts each
    traces = [torch.zeros(waves_max * 10, dtype=torch.int64, device=dev) for _ in range(launches)]
    launch(pkg, act, layers[0], out)
    torch.cuda.synchronize()

    def body():
        for r in range(launches):
            os.environ["WOQ_TRACE_PTR"] = hex(traces[r].data_ptr())
            launch(pkg, act, layers[r % copies], out)
    _, sec, _ = time_graph(body, launches, repeats=3)
    os.environ.pop("WOQ_TRACE_PTR", None)
    launched = last_launch(pkg)
    if not launched.startswith("stream row") or not bool((traces[3] != 0).any()):
        sys.exit("bench.py --mode timeline: no stamps were written - run it on a shape the row kernel serves, with "
                 "WOQ_LIB_PATH pointing at the library built by `python tensorrt-llm_amd/build.py --timeline`")
    stamps = {"wavefront starts": 0, "activations and weights requested": 1, "scales and zeros requested": 2,
              "arithmetic done": 6, "sums in LDS": 7, "barrier passed": 8, "wavefront ends": 9}
    per = {nm: [] for nm in stamps}
    next_start, life = [], []
    for r in range(2, launches - 1):
        t = traces[r].cpu().numpy().reshape(-1, 10)
        t = t[t[:, 0] != 0]
        t0 = t[:, 0].min()
        for nm, i in stamps.items():
            per[nm].append([np.percentile((t[:, i] - t0) / 100.0, q) for q in (0, 10, 50, 90, 99, 100)])
        nxt = traces[r + 1].cpu().numpy().reshape(-1, 10)
        next_start.append((nxt[nxt[:, 0] != 0][:, 0].min() - t0) / 100.0)
        life.append(float(np.median((t[:, 9] - t[:, 0]) / 100.0)))
    line = {"mode": "timeline", "shape": shape or "8b_gate_up", "k": k, "n": n, "kernel": launched,
            "us_per_launch_with_stamps": round(sec / launches * 1e6, 2), "wavefronts": int(t.shape[0]),
            "percentiles": ["min", "p10", "p50", "p90", "p99", "max"],
            "us_after_first_wavefront_start": {nm: [round(float(x), 2) for x in np.median(np.array(v), axis=0)]
                                               for nm, v in per.items()},
            "next_launch_first_wavefront_us": round(float(np.median(next_start)), 2),
            "wavefront_life_median_us": round(float(np.median(life)), 2)}
    print(json.dumps(line))


def run_operands(pkg, dev, m=4096, reps=20):
    """The real prefill kernels (W4A16 g128 bf16 and W4A8 on the 8B gate_up at M = 4096) on three sets of
    operands: the benchmark's random ones, the same weights with all-zero activations, and all-zero activations
    with weights whose stored bytes are all equal (every nibble 8: q = 0).  The instruction stream is the same
    in all three; what differs is the switching activity in the matrix core and with it the clock the power
    management sustains.  One JSON line."""
    name, k, n = SHAPES_8B[2]
    layer = make_layer(pkg, dev, k, n, 3000)
    flat = dict(layer)
    flat["weight"] = torch.full_like(layer["weight"], 0x88 - 256 if layer["weight"].dtype == torch.int8 else 0x88)
    g = torch.Generator(device=dev).manual_seed(3999)
    act_r = torch.randn((m, k), generator=g, device=dev).to(torch.bfloat16)
    act_0 = torch.zeros_like(act_r)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    line = {"mode": "operands", "shape": name, "m": m, "w4a16": {}, "w4a8": {}}
    for label, act, lay in [("random", act_r, layer), ("zero_activations", act_0, layer),
                            ("zero_activations_flat_weights", act_0, flat)]:
        launch(pkg, act, lay, out)
        torch.cuda.synchronize()
        _, sec, launches = time_graph(lambda: [launch(pkg, act, lay, out) for _ in range(reps)], reps, repeats=3)
        tf = 2.0 * m * n * k / (sec / launches) / 1e12
        line["w4a16"][label] = {"us": round(sec / launches * 1e6, 1), "tflops": round(tf, 1),
                                "frac_of_bf16_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4)}
    line["w4a16"]["kernel"] = last_launch(pkg)
    F = pkg.functional
    scales16 = layer["scales"].to(torch.float16)
    a8_r = (torch.randn((m, k), generator=g, device=dev) * 0.5).to(torch.float8_e4m3fn)
    a8_0 = torch.zeros_like(a8_r)
    for label, act, lay in [("random", a8_r, layer), ("zero_activations", a8_0, layer),
                            ("zero_activations_flat_weights", a8_0, flat)]:
        def run():
            F.woq_matmul_raw(act, None, lay["weight"], scales16, None, None, n=n, k=k, group_size=GROUP,
                             quant_algo=F.FP8_ALPHA, alpha=0.5, out_dtype=torch.bfloat16, out=out)
        run()
        torch.cuda.synchronize()
        _, sec, launches = time_graph(lambda: [run() for _ in range(reps)], reps, repeats=3)
        tf = 2.0 * m * n * k / (sec / launches) / 1e12
        line["w4a8"][label] = {"us": round(sec / launches * 1e6, 1), "tflops": round(tf, 1),
                               "frac_of_fp8_peak": round(tf / MFMA_FP8_PEAK_TFLOPS, 4)}
    line["w4a8"]["kernel"] = last_launch(pkg)
    print(json.dumps(line))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-gemm", action="store_true", help="skip the M=4096 extra")
    ap.add_argument("--replay-ms", type=int, default=0,
                    help="counter / trace modes: afterwards replay the launches from a HIP graph for this long")
    ap.add_argument("--summarize-trace", default=None, metavar="CSV",
                    help="print per-kernel durations of a rocprofv3 kernel trace (no GPU needed) and exit")
    ap.add_argument("--shape", default=None, help="gemm<M> and w4a8_<M> modes: the layer shape (8b_qkv ... 70b_down; default 8b_gate_up)")
    ap.add_argument("--mode", choices=["bench", "dominant", "dominant70b", "copy", "gemm4096", "gemm256", "gemm128", "gemm64", "gemm32", "gemm16", "gemm8", "gemm4", "w4a8_4096", "w4a8_256", "w4a8_64", "w4a8_16", "w4a8_8", "w4a8_decode", "moe_decode",
                                       "sweep", "ceilings", "operands", "timeline"],
                    default="bench", help="dominant / copy / gemm<M>: launch only that kernel, for rocprofv3 runs; "
                                          "sweep: the table named by --sweep")
    ap.add_argument("--sweep", choices=sorted(SWEEPS) + ["moe"], default="llama70b")
    ap.add_argument("--tuned", action="store_true",
                    help="sweep: also profile each layer's tactics and time the tuned choices")
    args = ap.parse_args()
    if args.summarize_trace:
        summarize_trace(args.summarize_trace)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1): the op contains no communication, a "
                 "tensor-parallel model gives each GPU its own column or row slice of the weights")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the matmul has no CPU path")
    pkg = import_package()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.mode == "sweep":
        if args.sweep == "moe":
            run_moe_sweep(pkg, dev)
        else:
            run_sweep(pkg, dev, args.sweep, args.tuned)
        return
    if args.mode == "ceilings":
        run_ceilings(pkg, dev)
        return
    if args.mode == "operands":
        run_operands(pkg, dev)
        return
    if args.mode == "timeline":
        run_timeline(pkg, dev, args.shape)
        return
    if args.mode != "bench":
        run_for_counters(pkg, dev, args.mode, shape=args.shape, replay_ms=args.replay_ms)
        return
    r = bench_decode(pkg, dev, args.steps, args.warmup)
    sec_per_step = r["host_s"] / args.steps
    value = r["per_step_bytes"] / sec_per_step / 1e9
    achieved = r["dom_bytes"] / r["dom_dur"] / 1e9
    line = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Llama-3-8B decoder-layer linears (qkv, o_proj, gate_up, down), W4A16 g128 "
                               "bf16 scales+zeros, decode GEMV M=1; %d rotating weight copies" % r["copies"],
                   "m": 1, "group_size": GROUP, "weight_bits": 4},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": recorded_traffic_bytes(r["dom_launch"]),
                     "traffic_source": TRAFFIC_PROFILE,
                     "kernel": r["dom_launch"] + " (bf16 x int4 g128 + zeros) on gate_up K=4096 N=28672",
                     "bytes_per_launch": r["dom_bytes"], "us_per_launch": round(r["dom_dur"] * 1e6, 3)},
        "per_shape": r["per_shape"],
        "event_ms_per_step": round(r["ev_s"] / args.steps * 1e3, 5),
        # every timed replay follows SETTLE_S of untimed replays of the same graph (the clocks of a GPU that
        # was idle dip for 20-40 ms after load starts); the step's very first replay, by the events, for comparison
        "settle_ms": SETTLE_S * 1e3,
        "first_replay_ms_per_step": round(r["first_replay_s"] / args.steps * 1e3, 5),
    }
    if not args.no_gemm:
        line["gemm"] = bench_gemm(pkg, dev)
        line["w4a8"] = bench_w4a8(pkg, dev)
    if not args.no_cpu:
        line["cpu_baseline"] = bench_cpu_baseline(r["layers"], r["acts"])
    print(json.dumps(line))


if __name__ == "__main__":
    main()
