#!/usr/bin/env python3
"""Benchmark of the mapped-operation backend on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME]] [--no-cpu]

One "step" is one forward + backward pass of the large weighted mapped
convolution (configuration 4: x 8x128x256x512 -> 128 channels, K = 9, P = 4
bispherical interpolation points, float32), with every tensor already resident
in HBM.  The headline value is images per second over K timed steps.  The same
JSON line also carries, under "kernels", the achieved rate of every other hot
kernel (tangent-image gather / scatter, mapped max pool / unpool, icosphere
convolution and transposed convolution) against its roofline, the roofline
object of the dominant kernel and a CPU baseline measured in the same run.

Algorithmic bytes / flops per launch (what "achieved" divides by the measured
duration) are the minimal tensor traffic of each operator:
    gather   : image + map + output
    scatter  : input + map + output (+ one weight-sum plane when normalising)
    pool     : input + map + values + int64 indices;  unpool: grad_out + indices + map + grad_in
    conv     : 2 * Cout * Cin * K * OH*OW * B flops per contraction
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "spherical-package_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_FP32_TFLOPS = 157.3     # dense matrix fp32
MFMA_BF16_TFLOPS = 2500.0    # dense bf16


def _nbytes(*arrays):
    return float(sum(a.numel() * a.element_size() for a in arrays if a is not None))


class Timer:
    """HIP-event timing on torch's current stream (the stream every kernel of this
    library is launched on)."""

    def __init__(self, torch):
        self.torch = torch

    def run(self, fn, steps, warmup, reps=1):
        """Mean and minimum time of one call of fn over `steps` timed regions of `reps` calls
        each.  reps > 1 is for calls of a few tens of microseconds, where the event pair
        itself (a few microseconds of command processing between the marker and the kernel)
        would be a visible part of a region holding one call; the calls of a region are issued
        back to back on the stream, so a region's time over reps is what one launch takes."""
        t = self.torch
        for _ in range(warmup):
            fn()
        t.cuda.synchronize()
        evs = [(t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True))
               for _ in range(steps)]
        for a, b in evs:
            a.record()
            for _ in range(reps):
                fn()
            b.record()
        t.cuda.synchronize()
        ms = [a.elapsed_time(b) / reps for a, b in evs]
        return float(np.mean(ms)), float(np.min(ms))


def _measured_traffic(kernel):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, scaled by
    a copy kernel of known size); kept with the profile summaries, None when not measured."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f).get(kernel)


def _roof(bound, work, ms, traffic=None, peak=None):
    if bound == "hbm":
        peak = HBM_PEAK_GBS
        achieved = work / (ms * 1e-3) / 1e9
        unit = "GB/s"
    else:
        achieved = work / (ms * 1e-3) / 1e12
        unit = "TFLOP/s"
    return {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": traffic}


def _conv_entry_points(torch, ops, x, m, iw, w, b, g, K, interp, compute):
    """The three contractions of one mapped-convolution layer call as separate C-ABI
    launches (what the autograd function issues), for per-kernel timing."""
    from _spherical_distortion_ext import _capi
    B, Cin, H, W = x.shape
    Cout = w.shape[0]
    OH, OW = m.shape[:2]
    P = 0 if iw is None else int(iw.shape[-1])
    mode = {"native": _capi.SDK_COMPUTE_NATIVE, "bf16": _capi.SDK_COMPUTE_BF16,
            "split": _capi.SDK_COMPUTE_SPLIT}[compute]
    nws = _capi.load().sdk_mapped_conv_workspace_bytes(B, Cin, Cout, H, W, OH, OW, K, P, interp, 0, mode)
    ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=x.device)
    out = torch.empty(B, Cout, OH, OW, device=x.device)
    gi, gw = torch.empty_like(x), torch.empty_like(w)
    gb = torch.empty(Cout, device=x.device)
    p, s = ops._ptr, ops._stream(x)
    dims = (B, Cin, H, W, Cout, OH, OW, K, P, interp, 0, mode, s)
    # the layer's plan, built once per map as the operators do (steady state of a training run)
    plan, nplan = ops._conv_plan(x, m, iw, H, W, K, P, interp)
    if plan is None:
        return {
            "forward": lambda: _capi.call("sdk_mapped_conv_forward", p(x), p(m), p(iw), p(w),
                                          p(b), p(out), p(ws), nws, *dims),
            "backward_input": lambda: _capi.call("sdk_mapped_conv_backward_input", p(g), p(m),
                                                 p(iw), p(w), p(gi), p(ws), nws, *dims),
            "backward_weight": lambda: _capi.call("sdk_mapped_conv_backward_weight", p(g), p(m),
                                                  p(iw), p(x), p(gw), p(ws), nws, *dims),
            "bias_grad": lambda: _capi.call("sdk_bias_grad", p(g), p(gb), B, Cout, OH * OW, 0, s),
        }, (ws, out, gi, gw, gb)
    pl = (p(plan), nplan)
    return {
        "forward": lambda: _capi.call("sdk_mapped_conv_forward_planned", p(x), p(m), p(iw), p(w),
                                      p(b), p(out), p(ws), nws, *pl, *dims),
        "backward_input": lambda: _capi.call("sdk_mapped_conv_backward_input_planned", p(g), p(m),
                                             p(iw), p(w), p(gi), p(ws), nws, *pl, *dims),
        "backward_weight": lambda: _capi.call("sdk_mapped_conv_backward_weight_planned", p(g),
                                              p(m), p(iw), p(x), p(gw), p(ws), nws, *pl, *dims),
        "bias_grad": lambda: _capi.call("sdk_bias_grad", p(g), p(gb), B, Cout, OH * OW, 0, s),
    }, (ws, out, gi, gw, gb, plan)


def verify_conv4(torch, ops, cfg, t, compute):
    """Outside the timed loop: the very tensors and launch shapes that were timed, compared
    element-wise with the CPU oracle on sampled pixels (tests/sampled_parity.py: the oracle
    evaluates the full image through the map sliced to those pixels).  Forward on both polar
    row pairs, the seam columns and random pixels; grad_input, grad_weight and grad_bias for a
    grad_output that is zero elsewhere; grad_input of the dense grad_output on sampled image
    pixels.  Tolerances (max|a-b| / max|b|): forward 1e-5, backward 1e-4; 1e-2 with bf16
    operands."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import sampled_parity as sp
    from oracle import oracle
    chk = sp.ConvOracle(oracle, cfg, n_random=512, n_targets=256, seed=4)
    K, interp = cfg["kernel_size"], cfg["interp"]
    x, m, iw, w, b, g = t
    ops.set_conv_compute(compute)
    try:
        y = ops.mapped_conv_forward(x, m, iw, w, b, K, interp)
        gs = torch.from_numpy(chk.g_sparse).to(x.device)
        gi, gw, gb = ops.mapped_conv_backward(gs, m, iw, x, w, b, K, interp)
        err = {"forward": chk.check_forward(y)}
        err["grad_input"], err["grad_weight"], err["grad_bias"] = \
            chk.check_backward_sparse(gi, gw, gb)
        del gs, gi, gw, gb, y
        gi, _, _ = ops.mapped_conv_backward(g, m, iw, x, w, b, K, interp)
        err["grad_input_dense"] = chk.check_backward_dense(gi)
    finally:
        ops.set_conv_compute("native")
    fwd, bwd = (1e-2, 1e-2) if compute == "bf16" else (1e-5, 1e-4)
    ok = err["forward"] <= fwd and all(v <= bwd for k, v in err.items() if k != "forward")
    return {"verified": bool(ok), "pixels": int(len(chk.pix)), "targets": int(len(chk.targets)),
            "max_rel_err": {k: float("%.3g" % v) for k, v in err.items()},
            "tolerance": {"forward": fwd, "backward": bwd}}


def bench_conv4(torch, ops, timer, steps, warmup, compute="native", batch=8, verify=False):
    import workloads
    cfg = workloads.config4(batch=batch)
    dev = "cuda:0"
    x, m, iw, w, b, g = (torch.from_numpy(cfg[k]).to(dev) for k in
                         ("x", "sample_map", "interp_weights", "weight", "bias", "grad_output"))
    K, interp = cfg["kernel_size"], cfg["interp"]
    B, Cin, H, W = x.shape
    Cout = w.shape[0]
    OH, OW = m.shape[:2]
    flops = 2.0 * Cout * Cin * K * OH * OW * B
    # the split mode delivers fp32 results, so it is priced against the fp32 peak like native
    peak = MFMA_BF16_TFLOPS if compute == "bf16" else MFMA_FP32_TFLOPS
    # tensors one contraction reads and writes (float32 in HBM whatever the operand type)
    tensor_bytes = _nbytes(x) + _nbytes(g) + _nbytes(m) + _nbytes(iw) + _nbytes(w)
    extra = {}
    ops.set_conv_compute(compute)
    try:
        def step(mm=m):
            ops.mapped_conv_forward(x, mm, iw, w, b, K, interp)
            ops.mapped_conv_backward(g, mm, iw, x, w, b, K, interp)
        if compute == "native":
            # a step on a map the operators have not seen (its plans are built inside the
            # forward call), after the kernels themselves have run once on another map
            step()
            torch.cuda.synchronize()
            fresh = m.clone()
            ms_first, _ = timer.run(lambda: step(fresh), 1, 0)
            extra["first_call_ms"] = ms_first
            del fresh
        ms, ms_min = timer.run(step, steps, warmup)
        if compute == "native":
            ops.set_conv_plan_cache(False)       # every call rebuilds what it needs
            try:
                extra["ms_per_step_cache_off"], _ = timer.run(step, max(3, steps // 2), 1)
            finally:
                ops.set_conv_plan_cache(True)
            from _spherical_distortion_ext import _capi
            P = int(iw.shape[-1])
            extra["plan_bytes_reserved"] = int(_capi.load().sdk_mapped_conv_plan_bytes(
                H, W, OH, OW, K, P, interp, 0))
            extra["workspace_bytes_reserved"] = int(_capi.load().sdk_mapped_conv_workspace_bytes(
                B, Cin, Cout, H, W, OH, OW, K, P, interp, 0, 0))
    finally:
        ops.set_conv_compute("native")
    calls, keep = _conv_entry_points(torch, ops, x, m, iw, w, b, g, K, interp, compute)
    parts = {}
    for name, fn in calls.items():
        t, _ = timer.run(fn, max(3, steps // 2), 1)
        traffic = _measured_traffic("mapped_conv_" + name) if compute == "native" else None
        if name == "bias_grad":
            parts[name] = dict(ms=t, **_roof("hbm", _nbytes(g), t))
        elif compute == "bf16":
            # With float32 tensors in HBM a contraction moves 1.13 GB for 309 GFLOP: 273 FLOP
            # per byte, below the 312 at which the bf16 matrix peak and the HBM peak meet, so
            # the roofline that bounds this mode is HBM; the matrix-unit figure is kept beside it.
            parts[name] = dict(ms=t, **_roof("hbm", tensor_bytes, t),
                               mfma_bf16_frac=round(flops / (t * 1e-3) / 1e12 / peak, 4))
        else:
            parts[name] = dict(ms=t, **_roof("mfma", flops, t, traffic=traffic, peak=peak))
    del keep
    dominant = max(("forward", "backward_input", "backward_weight"), key=lambda n: parts[n]["ms"])
    check = verify_conv4(torch, ops, cfg, (x, m, iw, w, b, g), compute) if verify else None
    return {"ms_per_step": ms, "ms_min": ms_min, "images_per_s": B / (ms * 1e-3),
            "flops_per_contraction": flops, "parts": parts, "dominant": dominant,
            "verification": check, "extra": extra}


def bench_conv1(torch, ops, timer, steps, warmup):
    """Configuration 1 (x [1,3,64,128] -> 16 channels, bilinear, K = 9): 7 MFLOP and 2 MB, bound by
    launch latency, so it is reported in microseconds per call and not against a roofline."""
    import workloads
    cfg = workloads.config1()
    dev = "cuda:0"
    x, m, w, b, g = (torch.from_numpy(cfg[k]).to(dev) for k in
                     ("x", "sample_map", "weight", "bias", "grad_output"))
    K, interp = cfg["kernel_size"], cfg["interp"]
    ms_f, _ = timer.run(lambda: ops.mapped_conv_forward(x, m, None, w, b, K, interp), steps, warmup)

    def step():
        ops.mapped_conv_forward(x, m, None, w, b, K, interp)
        ops.mapped_conv_backward(g, m, None, x, w, b, K, interp)
    ms_s, _ = timer.run(step, steps, warmup)
    out = {"forward_us": round(ms_f * 1e3, 1), "forward_backward_us": round(ms_s * 1e3, 1)}
    # the same step captured into a HIP graph and replayed (the library launches kernels only and
    # allocates nothing, so a caller bound by launches can do this): time per replay
    try:
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        ms_g, _ = timer.run(graph.replay, steps, warmup)
        out["forward_backward_graph_replay_us"] = round(ms_g * 1e3, 1)
    except Exception as e:  # reported, not fatal: the eager figures above stand
        out["forward_backward_graph_replay_us"] = None
        out["graph_error"] = str(e)[:200]
    return {"conv1_latency": out}


def bench_resample2(torch, ops, timer, steps, warmup, reps=8):
    import workloads
    cfg = workloads.config2()
    dev = "cuda:0"
    x = torch.from_numpy(cfg["x"]).to(dev)
    m = torch.from_numpy(cfg["sample_map"]).to(dev)
    H, W = cfg["out_shape"]
    patches = ops.resample_from_map(x, m, None, 1)
    ms_g, _ = timer.run(lambda: ops.resample_from_map(x, m, None, 1), steps, warmup, reps=8)
    ms_s, _ = timer.run(lambda: ops.resample_to_map_normalized(patches, m, None, H, W, 1, 1e-12),
                        steps, warmup, reps=8)
    # what the tensor library's copy reaches on tensors of this size (x to a second buffer,
    # 50 MB moved): the rate a 20 us memory-bound call can be held against
    xc = torch.empty_like(x)
    ms_c, _ = timer.run(lambda: xc.copy_(x), steps, warmup, reps=8)
    copy_small = dict(ms=ms_c, **_roof("hbm", 2 * _nbytes(x), ms_c))
    del xc
    gather_bytes = _nbytes(x, m, patches)
    scatter_bytes = _nbytes(patches, m, x) + H * W * 4.0
    # the UV way back: every image pixel reads its face's patch at (u, v); and its adjoint
    quad = torch.from_numpy(cfg["quad_idx"]).to(dev)
    uv = torch.from_numpy(cfg["tex_uv"]).to(dev)
    B, C = x.shape[:2]
    NT, TP = m.shape[0], cfg["patch"]
    tex = patches.view(B, C, NT, TP, TP)
    ms_uf, _ = timer.run(lambda: ops.resample_from_uv_maps(tex, quad, uv, 1), steps, warmup, reps=8)
    ms_ub, _ = timer.run(lambda: ops.resample_to_uv_maps(x, quad, uv, NT, TP, TP, 1), steps,
                         warmup, reps=8)
    uv_bytes = _nbytes(tex, quad, uv, x)
    # the kernel map of configuration 4's image, generated on the device (bytes = the map)
    ms_map, _ = timer.run(lambda: ops.equirect_kernel_map(256, 512, 3, 3), steps, warmup, reps=8)
    map_bytes = 256 * 512 * 9 * 2 * 4.0
    # voting resample: a 13-class label image halved in size, four sources per output pixel
    gen = torch.Generator().manual_seed(7)
    labels = torch.randint(0, 13, (B, 1, H, W), generator=gen, dtype=torch.int64).to(dev)
    yy, xx = torch.meshgrid(torch.arange(H) // 2, torch.arange(W) // 2, indexing="ij")
    vmap = torch.stack([xx, yy], -1).contiguous().to(dev)
    ms_v, _ = timer.run(lambda: ops.voting_resample_to_map(labels, vmap, H // 2, W // 2, 13),
                        steps, warmup, reps=8)
    vote_bytes = _nbytes(labels, vmap) + B * (H // 2) * (W // 2) * 8.0
    return {"copy_reference_50MB": copy_small,
            "voting_resample": dict(ms=ms_v, **_roof("hbm", vote_bytes, ms_v)),
            "map_generation": dict(ms=ms_map, **_roof("hbm", map_bytes, ms_map)),
            "uv_gather": dict(ms=ms_uf, **_roof("hbm", uv_bytes, ms_uf,
                                                traffic=_measured_traffic("resample_from_uv_maps"))),
            "uv_scatter": dict(ms=ms_ub, **_roof("hbm", uv_bytes, ms_ub,
                                                 traffic=_measured_traffic("resample_to_uv_maps"))),
            "gather": dict(ms=ms_g, **_roof("hbm", gather_bytes, ms_g,
                                            traffic=_measured_traffic("resample_from_map"))),
            "scatter_normalise": dict(ms=ms_s, **_roof("hbm", scatter_bytes, ms_s,
                                                       traffic=_measured_traffic("resample_to_map")))}


def bench_pool3(torch, ops, timer, steps, warmup, reps=8, with_cold=True):
    import workloads
    cfg = workloads.config3()
    dev = "cuda:0"
    x = torch.from_numpy(cfg["x"]).to(dev)
    m = torch.from_numpy(cfg["sample_map"]).to(dev)
    g = torch.from_numpy(cfg["grad_output"]).to(dev)
    K = cfg["kernel_size"]
    H, W = x.shape[2:]
    val, idx = ops.mapped_max_pool(x, m, None, K, 0)
    ms_f, _ = timer.run(lambda: ops.mapped_max_pool(x, m, None, K, 0), steps, warmup, reps=8)
    ms_b, _ = timer.run(lambda: ops.mapped_max_unpool(g, idx, m, None, H, W, K, 0), steps, warmup, reps=8)
    fwd_bytes = _nbytes(x, m, val, idx)
    bwd_bytes = _nbytes(g, idx, m, x)
    # average pooling on the same input and map: no index tensor on either side
    ms_af, _ = timer.run(lambda: ops.mapped_avg_pool(x, m, None, K, 0), steps, warmup, reps=8)
    ms_ab, _ = timer.run(lambda: ops.mapped_avg_unpool(g, m, None, H, W, K, 0), steps, warmup, reps=8)
    avg_bytes = _nbytes(x, m, val)
    # what a plain copy of the same input reaches on this GPU (the tensor library's copy kernel,
    # read + write): the rate a memory-bound kernel can be held against beside the published peak
    y = torch.empty_like(x)
    ms_c, _ = timer.run(lambda: y.copy_(x), steps, warmup, reps=8)
    del y
    # The same calls on tensors that are not in the 256 MB memory-side cache: six copies of the
    # inputs used in turn, the last six outputs kept alive so that every call writes fresh
    # memory too (2 to 3 GB per row).  `ms` above is the steady state of a loop over one set
    # of tensors, part of which the cache holds from call to call; `cold_ms` is what HBM gives.
    N = 6 if with_cold else 1
    xs = [x] + [x.clone() for _ in range(N - 1)]
    gs = [g] + [g.clone() for _ in range(N - 1)]
    idxs = [idx] + [idx.clone() for _ in range(N - 1)]

    def rotating(call):
        ring, turn = [None] * N, [0]

        def fn():
            k = turn[0] % N
            turn[0] += 1
            ring[k] = call(k)
        return fn
    cold = {}
    if with_cold:
        cold["pool_forward"], _ = timer.run(rotating(lambda k: ops.mapped_max_pool(xs[k], m, None, K, 0)),
                                            steps, warmup, reps=8)
        cold["pool_backward"], _ = timer.run(rotating(
            lambda k: ops.mapped_max_unpool(gs[k], idxs[k], m, None, H, W, K, 0)), steps, warmup, reps=8)
        cold["avg_pool_forward"], _ = timer.run(rotating(lambda k: ops.mapped_avg_pool(xs[k], m, None, K, 0)),
                                                steps, warmup, reps=8)
        cold["avg_pool_backward"], _ = timer.run(rotating(
            lambda k: ops.mapped_avg_unpool(gs[k], m, None, H, W, K, 0)), steps, warmup, reps=8)
        ys = [torch.empty_like(x) for _ in range(N)]
        cold["copy_reference"], _ = timer.run(rotating(lambda k: ys[k].copy_(xs[k])), steps, warmup, reps=8)
        del ys, xs, gs, idxs

    def row(name, ms_, nbytes, entry):
        d = dict(ms=ms_, **_roof("hbm", nbytes, ms_, traffic=_measured_traffic(entry) if entry else None))
        if with_cold:
            d["cold_ms"] = cold[name]
            d["cold_frac"] = round(nbytes / (cold[name] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        return d
    return {"copy_reference": row("copy_reference", ms_c, 2 * _nbytes(x), None),
            "pool_forward": row("pool_forward", ms_f, fwd_bytes, "mapped_max_pool"),
            "pool_backward": row("pool_backward", ms_b, bwd_bytes, "mapped_max_unpool"),
            "avg_pool_forward": row("avg_pool_forward", ms_af, avg_bytes, "mapped_avg_pool"),
            "avg_pool_backward": row("avg_pool_backward", ms_ab, avg_bytes, "mapped_avg_unpool"),
            "no_winner_outputs": int((idx < 0).sum().item())}


def bench_ico5(torch, ops, timer, steps, warmup):
    import workloads
    cfg = workloads.config5()
    dev = "cuda:0"
    t = {k: torch.from_numpy(v).to(dev) for k, v in cfg.items() if isinstance(v, np.ndarray)}
    K = cfg["kernel_size"]
    B, C, _, V = t["x"].shape
    flops = 2.0 * C * C * K * V * B

    def conv_step():
        ops.mapped_conv_forward(t["x"], t["sample_map"], None, t["weight"], t["bias"], K, 0)
        ops.mapped_conv_backward(t["grad_output"], t["sample_map"], None, t["x"], t["weight"],
                                 t["bias"], K, 0)
    ms_c, _ = timer.run(conv_step, steps, warmup)
    oh, ow = cfg["out_hw"]
    Vc = t["x_coarse"].shape[3]
    ms_t, _ = timer.run(lambda: ops.mapped_transposed_conv_forward(
        t["x_coarse"], t["up_map"], None, t["up_weight"], t["up_bias"], oh, ow, K, 0), steps,
        warmup)
    tflops = 2.0 * C * C * K * Vc * B
    # the same two workloads in the split compute mode (float32 results, bf16 matrix unit)
    ops.set_conv_compute("split")
    try:
        ms_cs, _ = timer.run(conv_step, steps, warmup)
        ms_ts, _ = timer.run(lambda: ops.mapped_transposed_conv_forward(
            t["x_coarse"], t["up_map"], None, t["up_weight"], t["up_bias"], oh, ow, K, 0), steps,
            warmup)
    finally:
        ops.set_conv_compute("native")
    return {"icosphere_conv_fwd_bwd_split": dict(ms=ms_cs, images_per_s=B / (ms_cs * 1e-3),
                                                 **_roof("mfma", 3 * flops, ms_cs,
                                                         peak=MFMA_FP32_TFLOPS)),
            "transposed_conv_forward_split": dict(ms=ms_ts, **_roof("mfma", tflops, ms_ts,
                                                                    peak=MFMA_FP32_TFLOPS)),
            "icosphere_conv_fwd_bwd": dict(ms=ms_c, images_per_s=B / (ms_c * 1e-3),
                                           **_roof("mfma", 3 * flops, ms_c,
                                                   peak=MFMA_FP32_TFLOPS)),
            "transposed_conv_forward": dict(ms=ms_t, **_roof("mfma", tflops, ms_t,
                                                             peak=MFMA_FP32_TFLOPS))}


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.lower().startswith("model name"):
                    return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(budget_s=12.0):
    """Times the CPU checker on a bounded sample of configuration 4 and reports images per
    second: whole batch-1 images (forward + backward) repeated for about `budget_s` seconds
    with the compiled reference, or one band of output rows, scaled, with the slower port."""
    import torch
    import workloads
    from oracle import oracle as orc
    try:
        from oracle import ref
        R = ref.load() if ref.available() else None
    except Exception:
        R = None
    H = 256
    cfg = workloads.config4(batch=1)
    K = 9
    if R is not None:
        tt = [torch.from_numpy(cfg[k]) for k in ("x", "sample_map", "interp_weights", "weight",
                                                 "bias", "grad_output")]
        it = R.InterpolationType(2)
        mod = R._weighted_mapped_convolution

        def one():
            mod.weighted_mapped_conv_forward(tt[0], tt[1], tt[2], tt[3], tt[4], K, it)
            mod.weighted_mapped_conv_backward(tt[5], tt[1], tt[2], tt[0], tt[3], tt[4], K, it)
        one()  # warm-up
        reps, t0 = 0, time.time()
        while reps < 1 or (time.time() - t0 < budget_s and reps < 16):
            one()
            reps += 1
        dt = time.time() - t0
        return {"value": round(reps / dt, 4), "unit": "images/s",
                "cores": int(torch.get_num_threads()), "cpu": _cpu_model(), "kind": "reference",
                "sample": "configuration 4 at batch 1 (one 128x256x512 image, fwd+bwd), %d "
                          "repetitions in %.1f s after one warm-up" % (reps, dt)}
    rows = 64
    m = np.ascontiguousarray(cfg["sample_map"][:rows])
    iw = np.ascontiguousarray(cfg["interp_weights"][:rows])
    g = np.ascontiguousarray(cfg["grad_output"][:, :, :rows])
    t0 = time.time()
    orc.mapped_conv_forward(cfg["x"], m, cfg["weight"], cfg["bias"], K, 2, iw)
    orc.mapped_conv_backward(g, m, cfg["x"], cfg["weight"], cfg["bias"], K, 2, iw)
    dt = time.time() - t0
    return {"value": round(rows / float(H) / dt, 4), "unit": "images/s",
            "cores": int(orc.num_threads()), "cpu": _cpu_model(), "kind": "port",
            "sample": "configuration 4, batch 1, output rows 0..%d of %d (%.1f s of CPU work), "
                      "fwd+bwd, scaled by the pixel share" % (rows - 1, H, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", default="", help="comma list of: conv4,conv4_bf16,conv4_split,conv1,resample2,pool3,ico5")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-cold", action="store_true",
                    help="skip the second series of the pooling rows (tensors the cache does not hold)")
    ap.add_argument("--no-verify", action="store_true",
                    help="skip the oracle check of the timed configuration after the timed loop")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (--gpus 1); "
                 "the path shards over the batch (only grad_weight / grad_bias would need an "
                 "all-reduce), which is not built")

    import torch
    from _spherical_distortion_ext import _ops as ops
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    timer = Timer(torch)
    only = [s for s in args.only.split(",") if s]
    want = lambda n: not only or n in only  # noqa: E731

    kernels = {}
    head = None
    if want("conv4"):
        head = bench_conv4(torch, ops, timer, args.steps, args.warmup,
                           verify=not args.no_verify)
        kernels["conv4_fp32"] = dict(ms_per_step=head["ms_per_step"],
                                     images_per_s=head["images_per_s"], **head["parts"],
                                     **head["extra"])
        torch.cuda.empty_cache()
    if want("conv4_bf16"):
        try:
            r = bench_conv4(torch, ops, timer, args.steps, args.warmup, compute="bf16")
            kernels["conv4_bf16"] = dict(ms_per_step=r["ms_per_step"],
                                         images_per_s=r["images_per_s"], **r["parts"])
        except RuntimeError as e:
            kernels["conv4_bf16"] = {"error": str(e)[:200]}
        torch.cuda.empty_cache()
    if want("conv4_split"):
        # float32 accuracy from the bf16 matrix unit (operands split into three bf16 pieces);
        # reported beside the headline, which stays the native fp32 arithmetic
        r = bench_conv4(torch, ops, timer, args.steps, args.warmup, compute="split")
        kernels["conv4_split"] = dict(ms_per_step=r["ms_per_step"],
                                      images_per_s=r["images_per_s"], **r["parts"])
        torch.cuda.empty_cache()
    if want("conv1"):
        kernels.update(bench_conv1(torch, ops, timer, max(args.steps, 20), args.warmup + 3))
    if want("resample2"):
        kernels.update(bench_resample2(torch, ops, timer, max(args.steps, 20), args.warmup + 3))
    if want("pool3"):
        kernels.update(bench_pool3(torch, ops, timer, max(args.steps, 20), args.warmup + 3,
                                   with_cold=not args.no_cold))
        torch.cuda.empty_cache()
    if want("ico5"):
        kernels.update(bench_ico5(torch, ops, timer, args.steps, args.warmup))
        torch.cuda.empty_cache()

    line = {"metric": "mapped_conv_fwd_bwd_images_per_sec", "unit": "images/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "configuration 4: weighted (P=4) bispherical mapped convolution "
                                   "fwd+bwd, x 8x128x256x512 -> 128 channels, K=9, float32",
                       "global_batch": 8}}
    if head is not None:
        dom = head["parts"][head["dominant"]]
        roof = {k: dom[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
        roof["kernel"] = "mapped_conv_" + head["dominant"]
        roof["traffic"] = _measured_traffic(roof["kernel"])
        line.update(value=round(head["images_per_s"], 3), ms_per_step=round(head["ms_per_step"], 4),
                    roofline=roof)
        # what the steady-state figure leaves out: the first step on a map (plans built),
        # a step with the plan cache off, and the memory the plans and the workspace reserve
        for key in ("first_call_ms", "ms_per_step_cache_off", "plan_bytes_reserved",
                    "workspace_bytes_reserved"):
            if key in head["extra"]:
                v = head["extra"][key]
                line[key] = round(v, 4) if isinstance(v, float) else v
        if head["verification"] is not None:
            line.update(verified=head["verification"]["verified"],
                        verification=head["verification"])
    else:
        line.update(value=None, ms_per_step=None, roofline=None)
    if "conv4_split" in kernels:
        # the same step with float32 results formed on the bf16 matrix unit (operands split
        # exactly into three bf16 pieces, fp32 accumulation, accuracy of the native mode);
        # `value` above stays on the native fp32 arithmetic
        line["split_compute"] = {"value": round(kernels["conv4_split"]["images_per_s"], 3),
                                 "unit": "images/s",
                                 "ms_per_step": round(kernels["conv4_split"]["ms_per_step"], 4),
                                 "dtype": "f32 operands as 3 bf16 pieces, 6 products, f32 accumulate"}
    line["cpu_baseline"] = None if args.no_cpu else cpu_baseline()
    line["kernels"] = kernels
    print(json.dumps(line))


if __name__ == "__main__":
    main()
