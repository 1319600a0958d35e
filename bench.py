#!/usr/bin/env python3
"""Benchmark of the Q8_0 matrix-product hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one pass of the hot path over one batch of synthetic input: the
full Qwen3-0.6B-shaped decode step at M = 1 (28 layers x {q, k, v, o, gate,
up, down} + lm_head = 197 Q8_0 GEMVs, 633 MB of weights), issued through the
C ABI as one dispatch group per step by the native step runner. Inputs are
resident in HBM before the timed region. One JSON line is printed:

  value      whole-step achieved bandwidth, algorithmic bytes / wall time
  roofline   the GEMV list kernel: algorithmic bytes per launch over its
             average launch duration (HIP events on the library's stream),
             beside the read bandwidth a read-only streaming kernel sustains
             on this box; and, as sub-objects, the other benchmark
             configurations, each against the peak of the unit it runs on and
             with its error against the CPU oracle:
               gemm_m512  the seven projections at 512 tokens (config 2)
               gemma      Gemma-3-1B shapes at 1 and 512 tokens (config 3)
               sweep_2b   2B-class shapes, 1..2048 tokens, f32 and int8
                          activations (config 4)
  cpu_baseline  the scalar CPU oracle timed on this host (reported only),
             with a bounded sample per configuration under per_config
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from tuckmill_amd import hip as H  # noqa: E402
from tuckmill_amd import synth as S  # noqa: E402

HBM_PEAK_GBS = 8000.0      # MI355X published HBM3E bandwidth
MFMA_F32_PEAK_TFLOPS = 157.3  # MI355X published dense f32 matrix rate
MFMA_I8_PEAK_TOPS = 5000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 matrix rate
# HBM bytes per launch of the decode step's GEMV list kernel, from the FETCH_SIZE and
# WRITE_SIZE counter runs summarised in profiles/gemv_list_kernel__decode_step__pmc_traffic.txt
# (fetch counter x 2.000 + write counter x 1.000, factors from a plain copy kernel).
DECODE_STEP_TRAFFIC_BYTES = 644.75e6
GEMMA_STEP_TRAFFIC_BYTES = 991.37e6  # the same for the Gemma-3-1B 79-GEMV step (its own profile file)
DECODE_STEP_TRAFFIC_SOURCE = ("constant from profiles/gemv_list_kernel__decode_step__pmc_traffic.txt "
                              "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --workload "
                              "traffic` on q8::gemv_list_kernel<1, 8, 1, true, 0, 224, false, false>); not "
                              "measured in this run")


class tmh_product(ctypes.Structure):
    _fields_ = [("w", ctypes.c_void_p), ("x", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("rows", ctypes.c_uint32), ("cols", ctypes.c_uint32), ("batch", ctypes.c_uint32),
                ("kind", ctypes.c_uint32)]


class tmh_timing(ctypes.Structure):
    _fields_ = [("wall_ms", ctypes.c_double), ("gpu_ms", ctypes.c_double),
                ("host_ms", ctypes.c_double), ("launches", ctypes.c_uint64),
                ("commits", ctypes.c_uint64), ("step_us_median", ctypes.c_double),
                ("step_us_min", ctypes.c_double), ("step_us_p10", ctypes.c_double),
                ("step_us_p90", ctypes.c_double)]


TMH_GEMV, TMH_GEMM, TMH_GEMM_MMA, TMH_GEMM_I8, TMH_QUANT = range(5)
TMH_RMSNORM, TMH_SILU_MUL, TMH_AXPY, TMH_ARGMAX, TMH_F16_GEMM, TMH_GELU_MUL = range(5, 11)
TMH_GEMM_I8_FMA = 11


def load_host():
    H.load_library()  # libtm_hip.so first, by absolute path
    path = os.path.join(ROOT, "tuckmill_amd", "libtm_host.so")
    if not os.path.exists(path):
        raise SystemExit(f"{path} is missing: run `python -m tuckmill_amd.build` first")
    lib = ctypes.CDLL(path)
    lib.tmh_run_steps.restype = ctypes.c_int
    lib.tmh_run_steps.argtypes = [ctypes.c_void_p, ctypes.POINTER(tmh_product), ctypes.c_uint32,
                                  ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int,
                                  ctypes.POINTER(tmh_timing), ctypes.c_char_p, ctypes.c_size_t]
    return lib


def _run(host, ctx, arr, n, warmup, steps, mode) -> tmh_timing:
    t = tmh_timing()
    err = ctypes.create_string_buffer(H.ERR_CAP)
    rc = host.tmh_run_steps(ctx.raw, arr, n, warmup, steps, mode, ctypes.byref(t), err, H.ERR_CAP)
    if rc != 0:
        raise SystemExit(f"step runner failed ({rc}): {err.value.decode()}")
    return t


# Preconditioning: after an idle period (weight synthesis on the host, a fence, a
# download) the first launches run up to 20 % slower while clocks and power ramp,
# for about 15 ms. Untimed windows of steps are run until three consecutive windows
# agree within 1 % on the GPU time per step, independent of --warmup.
PRECONDITION = {"window_ms": 5.0, "agree": 0.01, "windows_in_a_row": 3, "max_ms": 1500.0}


def precondition(host, ctx, arr, n, mode):
    t = _run(host, ctx, arr, n, 0, 2, mode)
    step_ms = max(t.gpu_ms / 2, 1e-3)
    per_window = int(min(50, max(3, round(PRECONDITION["window_ms"] / step_ms))))
    history, spent, windows = [], t.gpu_ms, 0
    while spent < PRECONDITION["max_ms"]:
        t = _run(host, ctx, arr, n, 0, per_window, mode)
        windows += 1
        spent += t.wall_ms
        history.append(t.gpu_ms / per_window)
        last = history[-PRECONDITION["windows_in_a_row"]:]
        if len(last) == PRECONDITION["windows_in_a_row"] and \
                max(last) - min(last) <= PRECONDITION["agree"] * min(last):
            return {"steps": 2 + windows * per_window, "windows": windows,
                    "steps_per_window": per_window, "stable": True, "ms": spent}
    return {"steps": 2 + windows * per_window, "windows": windows, "steps_per_window": per_window,
            "stable": False, "ms": spent}


def run_steps(host, ctx, products, warmup, steps, grouped=True, settle=True) -> tmh_timing:
    """`warmup` untimed steps, then exactly `steps` timed ones. With `settle`, the
    untimed preconditioning windows run first; what they took is left in
    `run_steps.last_precondition`."""
    arr = (tmh_product * len(products))(*products)
    mode = 2 if grouped == "recorded" else (1 if grouped else 0)
    run_steps.last_precondition = precondition(host, ctx, arr, len(products), mode) if settle \
        else None
    return _run(host, ctx, arr, len(products), warmup, steps, mode)


run_steps.last_precondition = None


def step_stats(t: tmh_timing, steps: int) -> dict:
    """Mean and order statistics of the GPU time per step (the commits' HIP events)."""
    out = {"mean_us": t.gpu_ms / steps * 1e3}
    if t.step_us_median > 0:
        out.update(median_us=t.step_us_median, min_us=t.step_us_min, p10_us=t.step_us_p10,
                   p90_us=t.step_us_p90)
    return out


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def decode_step_tensors():
    """(name, layer, rows, cols) of BASELINE config 1."""
    out = []
    for layer in range(S.QWEN3_0_6B_LAYERS):
        for name, rows, cols in S.QWEN3_0_6B_LAYER:
            out.append((name, layer, rows, cols))
    name, rows, cols = S.QWEN3_0_6B_LM_HEAD
    out.append((name, S.QWEN3_0_6B_LAYERS, rows, cols))
    return out


def build_decode_step(ctx, keep_host: bool, seal: bool = True):
    tensors = decode_step_tensors()
    products, keep, host_side = [], [], []
    for name, layer, rows, cols in tensors:
        seed = S.tensor_seed(1, layer, name)
        raw = S.make_weights(rows, cols, seed)
        x = S.make_activations(cols, seed)
        m = H.Matrix.load(ctx, raw, cols, rows, seal=seal)
        xb = ctx.buffer(cols * 4)
        xb.upload(0, x)
        yb = ctx.buffer(rows * 4)
        keep += [m, xb, yb]
        products.append(tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, 1, TMH_GEMV))
        if keep_host:
            host_side.append((raw, x, rows, cols, yb))
    return products, keep, host_side


def cpu_baseline(host_side, budget_s: float):
    """Times the scalar CPU oracle (single thread, like the reference's
    matvec loop) on whole decode steps until about `budget_s` seconds are
    spent, and checks the GPU's result of every product against it."""
    import oracle as O

    O.lib()
    step_bytes = sum(S.gemv_bytes(r, c) for _, _, r, c, _ in host_side)
    worst = 0.0
    gots = []
    t0 = time.perf_counter()
    for raw, x, rows, cols, yb in host_side:  # first pass doubles as the parity check
        want = O.gemv_q8_0_f32(raw, rows, cols, x, threads=1)
        got = yb.download_f32(0, rows)
        gots.append((got, want))
        worst = max(worst, float(np.max(np.abs(got - want)) / np.max(np.abs(want))))
    one = time.perf_counter() - t0
    # both against the exact (f64) sums, on the layer products of the first and the
    # last layer and the vocabulary projection
    gpu_f64 = cpu_f64 = 0.0
    for i in list(range(7)) + list(range(len(host_side) - 8, len(host_side))):
        raw, x, rows, cols, _ = host_side[i]
        exact = O.gemv_q8_0_f64(raw, rows, cols, x)
        scale = float(np.max(np.abs(exact)))
        gpu_f64 = max(gpu_f64, float(np.max(np.abs(gots[i][0] - exact)) / scale))
        cpu_f64 = max(cpu_f64, float(np.max(np.abs(gots[i][1] - exact)) / scale))
    reps = max(1, min(50, int(budget_s / max(one, 1e-3)) - 1))
    t0 = time.perf_counter()
    for _ in range(reps):
        for raw, x, rows, cols, _ in host_side:
            O.gemv_q8_0_f32(raw, rows, cols, x, threads=1)
    t1 = (time.perf_counter() - t0) / reps
    ncores = min(16, os.cpu_count() or 1)
    t0 = time.perf_counter()
    for raw, x, rows, cols, _ in host_side:
        O.gemv_q8_0_f32(raw, rows, cols, x, threads=ncores)
    tn = time.perf_counter() - t0
    return {
        "value": step_bytes / t1 / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{reps} full decode steps (197 GEMVs, {step_bytes} algorithmic bytes each) "
                  "through the scalar C restatement of kernels.rs:186-204, 1 thread",
        "ms_per_step": t1 * 1e3,
        "all_cores": {"value": step_bytes / tn / 1e9, "cores": ncores, "ms_per_step": tn * 1e3},
        "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
        "max_norm_err_gpu_vs_cpu": worst,
        "max_norm_err_gpu_vs_f64": gpu_f64, "max_norm_err_cpu_vs_f64": cpu_f64,
    }


def sample_tokens(M: int, n: int = 8) -> list:
    """Up to n token indices spread over 0..M-1, first and last included."""
    return sorted({int(v) for v in np.linspace(0, M - 1, min(n, M))})


def gemm_sample(raw, rows, cols, x_host, M, yb, tokens, int8=False, threads=None):
    """The sampled tokens of a product Y [M, rows] on the GPU and through the
    oracle (f32 activations: kernels.rs:186-204 per token; int8: quantize_row
    + kernels.rs:206-221), all rows. Returns (got, want, oracle_seconds)."""
    import oracle as O

    threads = threads or min(16, os.cpu_count() or 1)
    xs = np.ascontiguousarray(np.asarray(x_host).reshape(M, cols)[tokens]).reshape(-1)
    t0 = time.perf_counter()
    fn = O.gemm_q8_0_q8_0 if int8 else O.gemm_q8_0_f32
    want = fn(raw, rows, cols, xs, len(tokens), threads=threads)
    dt = time.perf_counter() - t0
    got = np.stack([yb.download_f32(t * rows, rows) for t in tokens])
    return got, want, dt


def norm_err(got, want) -> float:
    """max |got - want| / max |want| (the parity metric of the f32-activation kernels)."""
    scale = float(np.max(np.abs(want)))
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / (scale or 1.0))


def mfma_point(flops, t, steps, shapes, extra=None):
    """One timed prefill group against the peak of the matrix cores it ran on:
    the f32 cores (2*M*N*K over the time against 157.3 TFLOP/s) or, when the
    launch took the bf16 kernel (every activation as three exact bf16 pieces),
    the three bf16 products issued per f32 one against 2.5 PFLOP/s."""
    stats = step_stats(t, steps)
    us = stats.get("median_us") or stats["mean_us"]
    tile = H.gemm_mma_launch_tile(shapes)
    out = {"bound": "mfma", "us": us, "mean_us": stats["mean_us"],
           "launches_per_step": t.launches / steps, "tflops_f32_equivalent": flops / us / 1e6}
    if tile:
        out.update(kernel=f"q8::split_act_list_kernel + q8::gemm_bf16x3_kernel, tiles of {tile} tokens",
                   matrix_cores="bf16", achieved=3.0 * flops / us / 1e6, peak=MFMA_BF16_PEAK_TFLOPS)
    else:
        out.update(kernel="q8::gemm_mma kernels (v_mfma_f32_32x32x2_f32)", matrix_cores="f32",
                   achieved=flops / us / 1e6, peak=MFMA_F32_PEAK_TFLOPS)
    out["unit"] = "TFLOP/s"
    out["frac"] = out["achieved"] / out["peak"]
    if extra:
        out.update(extra)
    return out


def _layer_matrices(ctx, M, seal=True, keep_host=False):
    """The seven projection matrices of a Qwen3-0.6B layer, each with an X
    [M, K] and a Y [M, N] of its own: (products, buffers to free, by name)."""
    products, keep, mats = [], [], {}
    for name, rows, cols in S.QWEN3_0_6B_LAYER:
        raw = S.make_weights(rows, cols, S.tensor_seed(2, 0, name))
        m = H.Matrix.load(ctx, raw, cols, rows, seal=seal)
        xb = ctx.buffer(M * cols * 4)
        x = S.make_activations(M * cols, rows)
        xb.upload(0, x)
        yb = ctx.buffer(M * rows * 4)
        keep += [m.buf, xb, yb]
        mats[name] = (m, xb, yb, rows, cols) + ((raw, x) if keep_host else ())
        products.append(tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, M, TMH_GEMM_MMA))
    return products, keep, mats


def _group_err(mats, M, tokens):
    """Worst normalised error of the seven products' sampled tokens against the
    oracle, and the oracle's time for that sample (all host threads)."""
    worst, secs = 0.0, 0.0
    for name, _, _ in S.QWEN3_0_6B_LAYER:
        _, _, yb, rows, cols, raw, x = mats[name]
        got, want, dt = gemm_sample(raw, rows, cols, x[:M * cols], M, yb, tokens)
        worst = max(worst, norm_err(got, want))
        secs += dt
    return worst, secs


def _bench_layer_with_operators(host, ctx, mats, M, flops_total, steps, warmup, out, keep):
    """The layer as an executor encodes it, with the operators between the
    products (attention itself stands outside this path: o reads q's output):
    norm -> q,k,v -> o -> residual -> norm -> gate,up -> gated activation ->
    down -> residual, at M tokens and at the engine's prefill chunk of 128. The
    norms and the activation write the split form of their result themselves,
    the second norm takes the residual update in front of it."""
    hid, ffn = mats["q"][4], mats["gate"][3]
    bufs = {n: ctx.buffer(M * c * 4) for n, c in (("h", hid), ("xn", hid), ("xn2", hid), ("act", ffn))}
    wn = ctx.buffer(hid * 4)
    wn.upload(0, (1.0 + 0.1 * S.make_activations(hid, 11)).astype(np.float32))
    bufs["h"].upload(0, S.make_activations(M * hid, 12))
    def layer(tokens):
        def prod(name, x):
            m, _, yb, rows, cols = mats[name][:5]
            return tmh_product(m.buf.raw, x.raw, yb.raw, rows, cols, tokens, TMH_GEMM_MMA)
        return [tmh_product(wn.raw, bufs["h"].raw, bufs["xn"].raw, tokens, hid, tokens, TMH_RMSNORM),
                prod("q", bufs["xn"]), prod("k", bufs["xn"]), prod("v", bufs["xn"]),
                prod("o", mats["q"][2]),
                tmh_product(bufs["h"].raw, mats["o"][2].raw, bufs["h"].raw, 1, tokens * hid, 1, TMH_AXPY),
                tmh_product(wn.raw, bufs["h"].raw, bufs["xn2"].raw, tokens, hid, tokens, TMH_RMSNORM),
                prod("gate", bufs["xn2"]), prod("up", bufs["xn2"]),
                tmh_product(mats["gate"][2].raw, mats["up"][2].raw, bufs["act"].raw, 1, tokens * ffn, 1,
                            TMH_SILU_MUL),
                prod("down", bufs["act"]),
                tmh_product(bufs["h"].raw, mats["down"][2].raw, bufs["h"].raw, 1, tokens * hid, 1,
                            TMH_AXPY)]
    for key, tokens in (("layer_with_operators", M), ("layer_with_operators_m128", 128),
                        ("layer_with_operators_m256", 256)):
        if tokens > M:
            continue
        t = run_steps(host, ctx, layer(tokens), warmup, steps, grouped=True)
        stats = step_stats(t, steps)
        us = stats.get("median_us") or stats["mean_us"]
        out[key] = {
            "M": tokens, "us": us, "mean_us": stats["mean_us"], "us_per_token": us / tokens,
            "launches_per_step": t.launches / steps,
            "tflops_f32_equivalent": flops_total * tokens / M / us / 1e6,
            "order": "rmsnorm -> q,k,v -> o(q) -> axpy -> rmsnorm -> gate,up -> silu_mul -> down -> axpy; "
                     "no attention"}
    # Four such layers in one group at the engine's prefill chunk (the same weights four
    # times over: what a model's layers cost each when they follow one another, where the
    # residual update at the end of a layer rides in the next layer's first norm).
    if M >= 128:
        layers = 4
        t = run_steps(host, ctx, layer(128) * layers, warmup, max(steps // 2, 1), grouped=True)
        stats = step_stats(t, max(steps // 2, 1))
        us = stats.get("median_us") or stats["mean_us"]
        out["layer_chain_m128"] = {
            "M": 128, "layers": layers, "us": us, "us_per_layer": us / layers,
            "us_per_token": us / layers / 128,
            "launches_per_layer": t.launches / max(steps // 2, 1) / layers,
            "order": "four times (rmsnorm -> q,k,v -> o(q) -> axpy -> rmsnorm -> gate,up -> silu_mul -> down "
                     "-> axpy) in one group; no attention"}
    keep += list(bufs.values()) + [wn]


def bench_layer(host, ctx, steps, warmup):
    """Only the layer with its operators (for a kernel trace of just these launches)."""
    M = 512
    out = {"workload": "Qwen3-0.6B layer with its operators, 512, 256 and 128 tokens (no attention)", "M": M}
    products, keep, mats = _layer_matrices(ctx, M)
    flops_total = sum(2.0 * M * p.rows * p.cols for p in products)
    _bench_layer_with_operators(host, ctx, mats, M, flops_total, steps, warmup, out, keep)
    for b in keep:
        b.free()
    return out


def bench_gemm(host, ctx, steps, warmup, cpu=True, full=True):
    """BASELINE config 2: M = 512 tokens against the seven projection matrices
    of a Qwen3-0.6B layer, each with its own X [512, K]. One dispatch group over
    sealed weights (the seven independent products share one launch of the bf16
    kernel) and over weights as uploaded (the f32 matrix cores), each checked
    against the oracle on sampled tokens of every product; then one commit per
    product, the four dependent launches of a layer (q,k,v -> o -> gate,up ->
    down, each reading what the one before wrote), the layer with its operators,
    the engine's own prefill chunk of 128 tokens
    (crates/tuckcore/src/engine/metal.rs:25) and the vocabulary projection.
    Figures are medians over the timed steps where the commits could be told
    apart, means otherwise (method: crates/metal/src/tests.rs:1023-1073)."""
    M = 512
    out = {"config": "BASELINE config 2: seven Qwen3-0.6B projections, 512 tokens, f32 activations"}
    cpu_out = {}
    tokens = sample_tokens(M)
    products, keep, mats = _layer_matrices(ctx, M, keep_host=True)
    shapes = [(r, c, M) for _, r, c in S.QWEN3_0_6B_LAYER]
    flops_total = sum(2.0 * M * p.rows * p.cols for p in products)
    out["flops_per_step"] = flops_total
    t = run_steps(host, ctx, products, warmup, steps, grouped=True)
    err, secs = _group_err(mats, M, tokens)
    out["sealed_group"] = mfma_point(flops_total, t, steps, shapes, {
        "wall_us": t.wall_ms / steps * 1e3, "precondition_steps": run_steps.last_precondition["steps"],
        "max_norm_err_vs_cpu": err, "tokens_checked": len(tokens)})
    # the same seven products over weights as uploaded: the f32 matrix cores
    rproducts, rkeep, rmats = _layer_matrices(ctx, M, seal=False, keep_host=True)
    t = run_steps(host, ctx, rproducts, warmup, steps, grouped=True)
    rerr, _ = _group_err(rmats, M, tokens)
    out["raw_group"] = mfma_point(flops_total, t, steps, [], {
        "max_norm_err_vs_cpu": rerr, "tokens_checked": len(tokens),
        "weights_layout": "as uploaded (34-byte blocks)"})
    for b in rkeep:
        b.free()
    if cpu:
        import oracle as O
        # the oracle on the same sample: all threads (timed above), and one thread
        t0 = time.perf_counter()
        for name, _, _ in S.QWEN3_0_6B_LAYER:
            _, _, _, rows, cols, raw, x = mats[name]
            xs = np.ascontiguousarray(x.reshape(M, cols)[tokens[:2]]).reshape(-1)
            O.gemm_q8_0_f32(raw, rows, cols, xs, 2, threads=1)
        one = (time.perf_counter() - t0) / 2
        sample_flops = flops_total / M
        cpu_out = {"sample": f"{len(tokens)} of the 512 tokens x 7 projections through the scalar C "
                             "restatement (2 of them for the 1-thread figure)",
                   "ms_per_token_1_thread": one * 1e3, "gflops_1_thread": sample_flops / one / 1e9,
                   "ms_per_token_all_cores": secs / len(tokens) * 1e3,
                   "gflops_all_cores": sample_flops * len(tokens) / secs / 1e9,
                   "cores_all": min(16, os.cpu_count() or 1),
                   "ms_per_step_1_thread_extrapolated": one * M * 1e3}
    if full:
        us_sum, lone = 0.0, []
        for (name, rows, cols), p in zip(S.QWEN3_0_6B_LAYER, products):
            t = run_steps(host, ctx, [p], warmup, steps, grouped=False)
            pt = mfma_point(2.0 * M * rows * cols, t, steps, [(rows, cols, M)])
            us_sum += pt["us"]
            lone.append({"name": name, "rows": rows, "cols": cols, "us": pt["us"],
                         "matrix_cores": pt["matrix_cores"], "frac": pt["frac"]})
        out["one_commit_per_product"] = {"us": us_sum, "tflops_f32_equivalent": flops_total / us_sum / 1e6,
                                         "products": lone}
        # the same seven products wired as a layer: four launches, each behind the last
        h = mats["q"][1]
        dep = []
        for name, x in (("q", h), ("k", h), ("v", h), ("o", mats["q"][2]), ("gate", h), ("up", h),
                        ("down", mats["gate"][2])):
            m, _, yb, rows, cols = mats[name][:5]
            dep.append(tmh_product(m.buf.raw, x.raw, yb.raw, rows, cols, M, TMH_GEMM_MMA))
        t = run_steps(host, ctx, dep, warmup, steps, grouped=True)
        stats = step_stats(t, steps)
        us = stats.get("median_us") or stats["mean_us"]
        out["dependent_layer"] = {"us": us, "launches_per_step": t.launches / steps,
                                  "tflops_f32_equivalent": flops_total / us / 1e6,
                                  "order": "q,k,v -> o(q) -> gate,up -> down(gate); no attention"}
        _bench_layer_with_operators(host, ctx, mats, M, flops_total, steps, warmup, out, keep)
    # the engine's prefill chunk, one group, checked like the 512-token group
    m128 = [tmh_product(p.w, p.x, p.y, p.rows, p.cols, 128, TMH_GEMM_MMA) for p in products]
    t = run_steps(host, ctx, m128, warmup, steps, grouped=True)
    tok128 = sample_tokens(128)
    err128, _ = _group_err(mats, 128, tok128)
    out["m128_group"] = mfma_point(flops_total / 4, t, steps, [(r, c, 128) for r, c, _ in shapes], {
        "M": 128, "max_norm_err_vs_cpu": err128, "tokens_checked": len(tok128)})
    for b in keep:
        b.free()
    # The same model's vocabulary projection at M = 512 and at 64 tokens
    rows, cols = S.QWEN3_0_6B_LM_HEAD[1], S.QWEN3_0_6B_LM_HEAD[2]
    raw = S.make_weights(rows, cols, S.tensor_seed(2, 0, "lm_head"))
    m = H.Matrix.load(ctx, raw, cols, rows)
    xb = ctx.buffer(M * cols * 4)
    x = S.make_activations(M * cols, 5)
    xb.upload(0, x)
    yb = ctx.buffer(M * rows * 4)
    n = max(5, steps // 20)
    for key, mb in (("lm_head_m512", M), ("lm_head_m64", 64)):
        t = run_steps(host, ctx, [tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, mb, TMH_GEMM_MMA)],
                      max(2, warmup // 20), n, grouped=False)
        toks = sample_tokens(mb, 4)
        got, want, _ = gemm_sample(raw, rows, cols, x[:mb * cols], mb, yb, toks)
        out[key] = mfma_point(2.0 * mb * rows * cols, t, n, [(rows, cols, mb)], {
            "M": mb, "rows": rows, "cols": cols, "max_norm_err_vs_cpu": norm_err(got, want),
            "tokens_checked": len(toks)})
    for b in (m.buf, xb, yb):
        b.free()
    return out, cpu_out


def _weights_pool(ctx, shapes, copies, seed_base, keep_host=0):
    """`copies` distinct sealed weight sets of `shapes` [(name, rows, cols)];
    the raw bytes of the first `keep_host` entries stay on the host."""
    pool, host = [], []
    for c in range(copies):
        for name, rows, cols in shapes:
            raw = S.make_weights(rows, cols, seed_base + 17 * c + len(pool))
            if len(pool) < keep_host:
                host.append(raw)
            pool.append((name, rows, cols, H.Matrix.load(ctx, raw, cols, rows)))
    return (pool, host) if keep_host else pool


def hbm_point(abytes, us, extra=None):
    out = {"bound": "hbm", "us": us, "algorithmic_bytes": abytes, "achieved": abytes / us / 1e3,
           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": abytes / us / 1e3 / HBM_PEAK_GBS}
    if extra:
        out.update(extra)
    return out


def bench_gemma(host, ctx, steps, warmup, cpu=True):
    """BASELINE config 3: Gemma-3-1B shapes (hidden 1152 = 36 blocks per row,
    FFN 6912, lm_head 262144 x 1152). M = 1: a 26-layer FFN + lm_head step
    (79 GEMVs, 984 MB of weights) in one group, every product checked against the
    oracle. M = 512: the three FFN shapes in one group, and the lm_head on its
    own, sampled tokens checked."""
    import oracle as O

    out = {"config": "BASELINE config 3: Gemma-3-1B shapes, 1 and 512 tokens, f32 activations"}
    cpu_out = {}
    layers = 26
    ncores = min(16, os.cpu_count() or 1)
    ffn = [s for s in S.GEMMA3_1B if s[0] != "lm_head"]
    head = [s for s in S.GEMMA3_1B if s[0] == "lm_head"][0]
    pool, host_w = [], []
    for c in range(layers):
        for name, rows, cols in ffn:
            raw = S.make_weights(rows, cols, 3000 + 17 * c + len(pool))
            host_w.append(raw)
            pool.append((name, rows, cols, H.Matrix.load(ctx, raw, cols, rows)))
    raw = S.make_weights(head[1], head[2], 3999)
    host_w.append(raw)
    pool.append((head[0], head[1], head[2], H.Matrix.load(ctx, raw, head[2], head[1])))
    products, keep, host_x = [], [], []
    for name, rows, cols, m in pool:
        xb = ctx.buffer(cols * 4)
        x = S.make_activations(cols, rows + len(products))
        xb.upload(0, x)
        yb = ctx.buffer(rows * 4)
        keep += [xb, yb]
        host_x.append((x, yb))
        products.append(tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, 1, TMH_GEMV))
    step_bytes = sum(S.gemv_bytes(p.rows, p.cols) for p in products)
    t = run_steps(host, ctx, products, warmup, steps, grouped=True)
    stats = step_stats(t, steps)
    launch_us = t.gpu_ms * 1e3 / t.launches
    # parity of every product of the step; the all-cores pass is the CPU figure
    worst, t0 = 0.0, time.perf_counter()
    for (name, rows, cols, _), raw, (x, yb) in zip(pool, host_w, host_x):
        want = O.gemv_q8_0_f32(raw, rows, cols, x, threads=ncores)
        worst = max(worst, norm_err(yb.download_f32(0, rows), want))
    cpu_all = time.perf_counter() - t0
    out["gemv_step"] = hbm_point(step_bytes, launch_us, {
        "kernel": "q8::gemv_list_kernel (column tails 128 and 768)", "products": len(products),
        "launches_per_step": t.launches / steps, "median_us": stats.get("median_us"),
        "wall_us": t.wall_ms / steps * 1e3, "max_norm_err_vs_cpu": worst,
        "products_checked": len(products),
        "traffic": GEMMA_STEP_TRAFFIC_BYTES if t.launches == steps else None,
        "traffic_source": "constant from profiles/gemv_list_kernel__gemma3_1b_step__pmc_traffic.txt "
                          "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --workload "
                          "traffic`); not measured in this run"})
    head_p = products[-1]
    t = run_steps(host, ctx, [head_p], warmup, steps, grouped=False)
    us = t.gpu_ms / steps * 1e3
    out["lm_head_gemv"] = hbm_point(S.gemv_bytes(head_p.rows, head_p.cols), us,
                                    {"rows": head_p.rows, "cols": head_p.cols})
    if cpu:
        t0 = time.perf_counter()
        for (name, rows, cols, _), raw, (x, _) in list(zip(pool, host_w, host_x))[:6]:
            O.gemv_q8_0_f32(raw, rows, cols, x, threads=1)
        one = time.perf_counter() - t0
        six = sum(S.gemv_bytes(r, c) for _, r, c, _ in pool[:6])
        cpu_out = {"sample": "the 79-GEMV step once on all cores (the parity pass), two layers' FFN "
                             "matrices on 1 thread",
                   "gemv_step_ms_all_cores": cpu_all * 1e3, "gbs_all_cores": step_bytes / cpu_all / 1e9,
                   "cores_all": ncores, "gbs_1_thread": six / one / 1e9,
                   "gemv_step_ms_1_thread_extrapolated": step_bytes / (six / one) * 1e3}
    # M = 512
    M = 512
    gsteps, gwarm = max(5, steps // 4), max(2, warmup // 4)
    gp, gx = [], []
    for (name, rows, cols, m), raw in zip(pool[:3], host_w[:3]):
        xb = ctx.buffer(M * cols * 4)
        x = S.make_activations(M * cols, rows + 1)
        xb.upload(0, x)
        yb = ctx.buffer(M * rows * 4)
        keep += [xb, yb]
        gx.append((raw, rows, cols, x, yb))
        gp.append(tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, M, TMH_GEMM_MMA))
    flops = sum(2.0 * M * p.rows * p.cols for p in gp)
    t = run_steps(host, ctx, gp, gwarm, gsteps, grouped=True)
    toks = sample_tokens(M, 4)
    worst = 0.0
    for raw, rows, cols, x, yb in gx:
        got, want, _ = gemm_sample(raw, rows, cols, x, M, yb, toks)
        worst = max(worst, norm_err(got, want))
    out["ffn_gemm_m512"] = mfma_point(flops, t, gsteps, [(p.rows, p.cols, M) for p in gp], {
        "M": M, "max_norm_err_vs_cpu": worst, "tokens_checked": len(toks)})
    name, rows, cols, m = pool[-1]
    xb = ctx.buffer(M * cols * 4)
    x = S.make_activations(M * cols, 7)
    xb.upload(0, x)
    yb = ctx.buffer(M * rows * 4)
    keep += [xb, yb]
    flops = 2.0 * M * rows * cols
    n = max(5, steps // 20)
    t = run_steps(host, ctx, [tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, M, TMH_GEMM_MMA)],
                  2, n, grouped=False)
    got, want, secs = gemm_sample(host_w[-1], rows, cols, x, M, yb, toks)
    out["lm_head_gemm_m512"] = mfma_point(flops, t, n, [(rows, cols, M)], {
        "M": M, "rows": rows, "cols": cols, "max_norm_err_vs_cpu": norm_err(got, want),
        "tokens_checked": len(toks)})
    if cpu:
        cpu_out["lm_head_m512_ms_per_token_all_cores"] = secs / len(toks) * 1e3
    for b in keep:
        b.free()
    for _, _, _, m in pool:
        m.buf.free()
    return out, cpu_out


SWEEP_HEADLINE_M = (1, 8, 64, 512, 2048)  # the batches BASELINE config 4 names


def bench_sweep(host, ctx, steps, warmup, cpu=True, batches=None):
    """BASELINE config 4: 2B-class shapes (hidden 2048, FFN 6144), M in
    {1, 8, 64, 512, 2048} plus the small batches in between, f32 activations
    and the int8-activation profile.
    Each point runs over 20 distinct weight copies per shape (535 MB in all),
    so small M is measured against HBM, not against the caches. Every point
    carries both rooflines (algorithmic bytes against 8 TB/s, operations against
    the peak of the matrix cores the launch used) and its error against the
    oracle on sampled tokens of one copy of each shape (int8: bit equality)."""
    import oracle as O

    copies = 20
    pool, host_w = _weights_pool(ctx, list(S.SWEEP_2B), copies, 4000, keep_host=len(S.SWEEP_2B))
    wbytes = sum(S.q8_0_bytes(r, c) for _, r, c, _ in pool)
    out = {"config": "BASELINE config 4: 2B-class shapes (6144 x 2048, 2048 x 6144), "
                     f"{copies} copies of each = {len(pool)} products per step",
           "weights_bytes": wbytes, "points": []}
    maxM = 2048
    maxc = max(c for _, _, c, _ in pool)
    maxr = max(r for _, r, _, _ in pool)
    xb = ctx.buffer(maxM * maxc * 4)
    x_host = S.make_activations(maxM * maxc, 99)
    xb.upload(0, x_host)
    widths = sorted({c for _, _, c, _ in pool})
    xqs = {c: ctx.buffer(H.xq_bytes(c, maxM)) for c in widths}
    ys = [ctx.buffer(maxM * maxr * 4) for _ in pool]
    slice_x, slice_y, slice_host = [], [], []
    ncores = min(16, os.cpu_count() or 1)
    for M in (batches or (1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 2048)):
        n = max(10 if M < 64 else 5 if M < 512 else 3,
                steps // (10 if M < 64 else 200 if M < 512 else 1000))
        w = max(2, n // 5)
        flops = sum(2.0 * M * r * c for _, r, c, _ in pool)
        abytes = sum(S.q8_0_bytes(r, c) + 4 * M * c + 4 * M * r for _, r, c, _ in pool)
        paths = []
        if M == 1:
            paths.append(("f32 gemv", TMH_GEMV, M))
        if 1 < M <= 32:
            paths.append(("f32 gemm (gemv arithmetic)", TMH_GEMM, M))
        if 2 <= M <= 512:
            paths.append(("f32 mfma entry point", TMH_GEMM_MMA, M))
        if M > 512:
            paths.append(("f32 mfma entry point (slices of 512)", TMH_GEMM_MMA, 512))
        paths.append(("int8 activations", TMH_GEMM_I8, M))
        if M >= 5:
            paths.append(("int8 activations, fused tail", TMH_GEMM_I8_FMA, M))
        for label, kind, mb in paths:
            prods = []
            slices = (M + mb - 1) // mb
            quant_us = None
            if kind in (TMH_GEMM_I8, TMH_GEMM_I8_FMA):
                # activations are quantized once per distinct width (timed apart)
                qprods = [tmh_product(None, xb.raw, xqs[c].raw, 1, c, M, TMH_QUANT) for c in widths]
                tq = run_steps(host, ctx, qprods, 1, 3, grouped=True, settle=False)
                quant_us = tq.gpu_ms / 3 * 1e3
                for (name, r, c, m), yb in zip(pool, ys):
                    prods.append(tmh_product(m.buf.raw, xqs[c].raw, yb.raw, r, c, M, kind))
            else:
                # a batch above the largest one of a call goes in slices, each with
                # its own rows of X and of Y (buffers of their own here: the step
                # runner's products carry no offsets)
                while len(slice_x) < slices - 1:
                    sx = ctx.buffer(mb * maxc * 4)
                    sh = S.make_activations(mb * maxc, 100 + len(slice_x))
                    sx.upload(0, sh)
                    slice_x.append(sx)
                    slice_host.append(sh)
                    slice_y.append([ctx.buffer(mb * maxr * 4) for _ in pool])
                for i, ((name, r, c, m), yb) in enumerate(zip(pool, ys)):
                    prods.append(tmh_product(m.buf.raw, xb.raw, yb.raw, r, c, mb, kind))
                    for sl in range(slices - 1):
                        prods.append(tmh_product(m.buf.raw, slice_x[sl].raw, slice_y[sl][i].raw,
                                                 r, c, mb, kind))
            t = run_steps(host, ctx, prods, w, n, grouped=True)
            us = t.gpu_ms / n * 1e3
            # parity: sampled tokens of the first copy of each shape (for 2048 tokens in
            # slices: of the first and of the last slice)
            toks = sample_tokens(mb, 4)
            err, equal = 0.0, True
            for i, raw in enumerate(host_w):
                _, r, c, _ = pool[i]
                checks = [(x_host, ys[i])]
                if slices > 1:
                    checks.append((slice_host[slices - 2], slice_y[slices - 2][i]))
                for xh, yb in checks:
                    got, want, _ = gemm_sample(raw, r, c, xh[:mb * c], mb, yb, toks,
                                               int8=kind in (TMH_GEMM_I8, TMH_GEMM_I8_FMA),
                                               threads=ncores)
                    err = max(err, norm_err(got, want))
                    equal = equal and np.array_equal(got.view(np.uint32), want.view(np.uint32))
            pt = {"M": M, "path": label, "us": us, "launches": t.launches / n,
                  "gbs": abytes / us / 1e3, "frac_hbm": abytes / us / 1e3 / HBM_PEAK_GBS,
                  "tflops": flops / us / 1e6, "max_norm_err_vs_cpu": err}
            if kind in (TMH_GEMM_I8, TMH_GEMM_I8_FMA):
                pt.update(mfma_peak="int8 5.0 POP/s", frac_mfma=flops / us / 1e6 / MFMA_I8_PEAK_TOPS,
                          quantize_act_us=quant_us, bit_equal_to_cpu=bool(equal),
                          kernel="q8::gemv_i8_list_kernel (v_dot4)" if M <= 4
                          else "q8::gemm_i8_lds_kernel (v_mfma_i32_16x16x32_i8)")
            elif kind == TMH_GEMM_MMA and \
                    (mb >= 9 or all(H.gemm_mma_small_batch_on_tiles(r, c, mb) for _, r, c, _ in pool)) and \
                    H.gemm_mma_launch_tile([(r, c, mb) for _, r, c, _ in pool]):
                # three bf16 products are issued per f32 one
                pt.update(path=label + ": bf16 matrix cores, exact products",
                          mfma_peak="bf16 2.5 PFLOP/s",
                          frac_mfma=3.0 * flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS)
            elif kind == TMH_GEMM_MMA and mb > 16:
                pt.update(path=label + ": f32 matrix cores", mfma_peak="f32 157.3 TFLOP/s",
                          frac_mfma=flops / us / 1e6 / MFMA_F32_PEAK_TFLOPS)
            else:  # the vector kernels: f32 multiply-adds, no matrix cores
                pt.update(mfma_peak=None, frac_mfma=None)
            out["points"].append(pt)
    out["points"].sort(key=lambda pt: (pt["M"], pt["path"].startswith("int8")))
    # where the matrix cores take over from the vector (GEMV-arithmetic) kernels
    best = {}
    for pt in out["points"]:
        if pt["path"].startswith("int8"):
            continue
        cur = best.get(pt["M"])
        if cur is None or pt["us"] < cur["us"]:
            best[pt["M"]] = pt
    mfma_from = [M for M, pt in sorted(best.items()) if pt["frac_mfma"] is not None]
    hbm_to = [M for M, pt in sorted(best.items()) if pt["frac_hbm"] >= 0.5]
    out["crossover"] = {
        "fastest_f32_path_by_M": {str(M): pt["path"] for M, pt in sorted(best.items())},
        "matrix_cores_fastest_from_M": mfma_from[0] if mfma_from else None,
        "at_least_half_of_hbm_peak_up_to_M": hbm_to[-1] if hbm_to else None,
        "ridge_estimate": "2*M flops per weight byte x 34/32: the f32 vector rate (157 TFLOP/s) meets "
                          "8 TB/s near M = 10, the measured crossover is where the vector kernels' "
                          "issue rate, not HBM, starts to bound them"}
    cpu_out = {}
    if cpu:
        # one copy of each shape, one token: both oracles, one thread and all cores
        x1 = x_host[:maxc]
        res = {}
        for label, fn in (("f32", O.gemv_q8_0_f32), ("int8", O.gemv_q8_0_q8_0)):
            for th in (1, ncores):
                t0 = time.perf_counter()
                for i, raw in enumerate(host_w):
                    _, r, c, _ = pool[i]
                    fn(raw, r, c, x1[:c], threads=th)
                res[(label, th)] = time.perf_counter() - t0
        one_bytes = sum(S.gemv_bytes(pool[i][1], pool[i][2]) for i in range(len(host_w)))
        one_flops = sum(2.0 * pool[i][1] * pool[i][2] for i in range(len(host_w)))
        cpu_out = {"sample": "one copy of each of the two shapes, one token (the CPU path is a loop "
                             "of such GEMVs over tokens: forward.rs:703-735)",
                   "f32_ms_per_token_1_thread": res[("f32", 1)] * 1e3,
                   "f32_gbs_1_thread": one_bytes / res[("f32", 1)] / 1e9,
                   "f32_ms_per_token_all_cores": res[("f32", ncores)] * 1e3,
                   "int8_ms_per_token_1_thread": res[("int8", 1)] * 1e3,
                   "int8_gops_1_thread": one_flops / res[("int8", 1)] / 1e9,
                   "int8_ms_per_token_all_cores": res[("int8", ncores)] * 1e3,
                   "cores_all": ncores,
                   "step_of_40_products_ms_1_thread_extrapolated_per_token":
                       res[("f32", 1)] * copies * 1e3}
    for b in [xb] + list(xqs.values()) + ys + slice_x + [y for per in slice_y for y in per]:
        b.free()
    for _, _, _, m in pool:
        m.buf.free()
    return out, cpu_out


def read_ceiling(ctx, gib=1, reps=10):
    """The read bandwidth this box sustains for a kernel that does nothing but
    read: tm_hip_xor_checksum_u32 over `gib` GiB (non-temporal 16-byte loads, 8 KiB
    per wave at a time, 8 KiB written per launch), median of `reps` commits."""
    n = gib << 28  # 32-bit words
    if n >= 1 << 32:
        raise SystemExit("read_ceiling: at most 15 GiB")
    src, part = ctx.buffer(n * 4), ctx.buffer(H.CHECKSUM_PARTIAL_BYTES)
    ctx.fence()
    for _ in range(4):
        ctx.xor_checksum_u32(src, 0, n, part)
    ctx.fence()
    ctx.set_commit_log(True)
    for _ in range(reps):
        ctx.xor_checksum_u32(src, 0, n, part)
    ctx.fence()
    us = np.sort(np.asarray(ctx.read_commit_log(), dtype=np.float64)[-reps:]) / 1e3
    ctx.set_commit_log(False)
    src.free()
    part.free()
    med = float(np.median(us))
    return {"kernel": "q8::xor_checksum_kernel", "bytes_read": n * 4, "median_us": med,
            "min_us": float(us[0]), "gbs": n * 4 / med / 1e3, "gbs_best": n * 4 / float(us[0]) / 1e3,
            "frac_of_published_peak": n * 4 / med / 1e3 / HBM_PEAK_GBS}


def bench_f16(host, ctx, steps, warmup):
    """The F16 twins on the 2B-class projection shapes: 20 copies of each matrix as
    F16 (1.0 GB per pass), batch 1, 2, 4, 8 and 32, one commit per pass."""
    copies = 20
    rng = np.random.default_rng(7)
    mats = []
    for name, r, c in S.SWEEP_2B:
        h = (rng.standard_normal(r * c, dtype=np.float32) * np.float32(0.02)).astype(np.float16)
        for _ in range(copies):
            b = ctx.buffer(r * c * 2)
            b.upload(0, h.view(np.uint8))
            mats.append((r, c, b))
    wbytes = sum(r * c * 2 for r, c, _ in mats)
    maxc = max(c for _, c, _ in mats)
    maxr = max(r for r, _, _ in mats)
    xb = ctx.buffer(32 * maxc * 4)
    xb.upload(0, S.make_activations(32 * maxc, 98))
    ys = [ctx.buffer(32 * maxr * 4) for _ in mats]
    out = {"workload": "F16 twins, 2B-class shapes", "weights_bytes": wbytes, "points": []}
    for M in (1, 2, 4, 8, 32):
        n = max(3, steps // 10)
        prods = [tmh_product(b.raw, xb.raw, yb.raw, r, c, M, TMH_F16_GEMM)
                 for (r, c, b), yb in zip(mats, ys)]
        t = run_steps(host, ctx, prods, max(2, n // 5), n, grouped=True)
        us = t.gpu_ms / n * 1e3
        abytes = wbytes + sum(4 * M * (r + c) for r, c, _ in mats)
        out["points"].append({"M": M, "us": us, "launches": t.launches / n, "gbs": abytes / us / 1e3,
                              "pct_of_hbm_peak": abytes / us / 1e3 / 80.0})
    for b in [xb] + ys + [m[2] for m in mats]:
        b.free()
    return out


# (hidden, q width, k/v width, FFN width, vocabulary, layers, gated activation)
CHAIN_MODELS = {
    "qwen": ("Qwen3-0.6B", 1024, 2048, 1024, 3072, 151_936, S.QWEN3_0_6B_LAYERS, "silu"),
    "gemma": ("Gemma-3-1B", 1152, 1024, 256, 6912, 262_144, 26, "gelu_tanh"),
    "1.7b": ("Qwen3-1.7B", 2048, 2048, 1024, 6144, 151_936, 28, "silu"),
    # an 8 B-class model's widths (4096 hidden, 14336 FFN, grouped-query k/v of 1024), 8 of its
    # 32 layers so that the synthetic weights stay at 2.3 GB: launches of 18-125 MB each
    "8b": ("8B-class widths, 8 layers", 4096, 4096, 1024, 14336, 128_256, 8, "silu"),
}


def bench_chain(host, ctx, steps, warmup, recorded=True, model="qwen", tokens=1):
    """The decode step with its data dependencies: per layer rmsnorm -> q,k,v -> o ->
    residual -> rmsnorm -> gate,up -> silu_mul -> down -> residual, then final norm,
    lm_head and greedy argmax, Qwen3-0.6B shapes (or Gemma-3-1B's), one dispatch group per token
    (attention, RoPE and the KV cache are not part of this path: o reads q in place of
    the attention output, which has the same length and the same dependence). Products that do not depend on each other still share a launch (q,k,v and
    gate,up), everything else is ordered, so the step is bound by launch latency, not by
    HBM: this is the figure a graph replay or wider fusion would have to beat.
    `tokens` > 1: the same step over that many tokens with the exact small-batch GEMM
    (`q8_0_gemm`), the shape of a speculative step that verifies a draft with the
    decode arithmetic (crates/tuckcore/src/engine/metal.rs:2170-2192: two tokens);
    the operators run over `tokens` rows, the argmax over the first row."""
    T = int(tokens)
    model_name, hidden, qdim, kvdim, ffn, vocab, layers, act = CHAIN_MODELS[model]
    act_kind = TMH_SILU_MUL if act == "silu" else TMH_GELU_MUL
    keep, prods = [], []

    def fbuf(n, seed=None):
        b = ctx.buffer(n * 4)
        if seed is not None:
            b.upload(0, S.make_activations(n, seed))
        keep.append(b)
        return b

    def mat(rows, cols, seed):
        m = H.Matrix.load(ctx, S.make_weights(rows, cols, seed), cols, rows)
        keep.append(m)
        return m

    h, n, t = fbuf(T * hidden, 1), fbuf(T * hidden), fbuf(T * hidden)
    q, k, v = fbuf(T * qdim), fbuf(T * kvdim), fbuf(T * kvdim)
    gate, up = fbuf(T * ffn), fbuf(T * ffn)
    logits, partial, token = fbuf(T * vocab), ctx.buffer(H.ARGMAX_PARTIAL_BYTES), ctx.buffer(8)
    keep += [partial, token]
    wbytes = 0

    def product(m, x, y, rows, cols):
        nonlocal wbytes
        wbytes += S.gemv_bytes(rows, cols)
        prods.append(tmh_product(m.buf.raw, x.raw, y.raw, rows, cols, T,
                                 TMH_GEMV if T == 1 else TMH_GEMM))

    for layer in range(layers):
        g1, g2 = fbuf(hidden, 100 + layer), fbuf(hidden, 200 + layer)
        prods.append(tmh_product(g1.raw, h.raw, n.raw, T, hidden, 1, TMH_RMSNORM))
        product(mat(qdim, hidden, 5000 + 7 * layer), n, q, qdim, hidden)
        product(mat(kvdim, hidden, 5001 + 7 * layer), n, k, kvdim, hidden)
        product(mat(kvdim, hidden, 5002 + 7 * layer), n, v, kvdim, hidden)
        product(mat(hidden, qdim, 5003 + 7 * layer), q, t, hidden, qdim)
        prods.append(tmh_product(h.raw, t.raw, h.raw, 1, T * hidden, 1, TMH_AXPY))
        prods.append(tmh_product(g2.raw, h.raw, n.raw, T, hidden, 1, TMH_RMSNORM))
        product(mat(ffn, hidden, 5004 + 7 * layer), n, gate, ffn, hidden)
        product(mat(ffn, hidden, 5005 + 7 * layer), n, up, ffn, hidden)
        prods.append(tmh_product(gate.raw, up.raw, gate.raw, 1, T * ffn, 1, act_kind))
        product(mat(hidden, ffn, 5006 + 7 * layer), gate, t, hidden, ffn)
        prods.append(tmh_product(h.raw, t.raw, h.raw, 1, T * hidden, 1, TMH_AXPY))
    gf = fbuf(hidden, 999)
    prods.append(tmh_product(gf.raw, h.raw, n.raw, T, hidden, 1, TMH_RMSNORM))
    product(mat(vocab, hidden, 6000), n, logits, vocab, hidden)
    prods.append(tmh_product(partial.raw, logits.raw, token.raw, 1, vocab, 1, TMH_ARGMAX))
    ctx.fence()
    tg = run_steps(host, ctx, prods, warmup, steps, grouped=True)
    out = {"workload": f"{model_name} decode step with data dependencies (no attention)" +
                       (f", {T} tokens through the exact small-batch GEMM" if T > 1 else ""),
           "tokens": T,
           "operators_per_step": len(prods), "algorithmic_bytes": wbytes,
           "grouped": {"us": tg.wall_ms / steps * 1e3, "gpu_us": tg.gpu_ms / steps * 1e3,
                       "launches_per_step": tg.launches / steps,
                       "gbs": wbytes / (tg.wall_ms / steps * 1e-3) / 1e9,
                       "host_issue_us": tg.host_ms / steps * 1e3}}
    legs = [("grouped", True)]
    if recorded:
        tr = run_steps(host, ctx, prods, warmup, steps, grouped="recorded")
        out["recorded_step_replayed"] = {"us": tr.wall_ms / steps * 1e3,
                                         "gpu_us": tr.gpu_ms / steps * 1e3,
                                         "launches_per_step": tr.launches / steps,
                                         "gbs": wbytes / (tr.wall_ms / steps * 1e-3) / 1e9,
                                         "host_issue_us": tr.host_ms / steps * 1e3}
        legs.append(("recorded_step_replayed", "recorded"))
    # Over many steps the host is throttled by the depth of the hardware queue,
    # so its own cost per token is measured on a run short enough to fit.
    for name, mode in legs:
        ts = run_steps(host, ctx, prods, 2, 6, grouped=mode)
        out[name]["host_issue_us_short_run"] = ts.host_ms / 6 * 1e3
    n_un = max(10, steps // 10)
    tu = run_steps(host, ctx, prods, 3, n_un, grouped=False)
    out["one_commit_per_operator"] = {"us": tu.wall_ms / n_un * 1e3,
                                      "launches_per_step": tu.launches / n_un,
                                      "gbs": wbytes / (tu.wall_ms / n_un * 1e-3) / 1e9}
    for obj in keep:
        (obj.buf if isinstance(obj, H.Matrix) else obj).free()
    return out


def run_traffic(host, ctx):
    """A short, fixed sequence for hardware-counter runs (rocprofv3 --pmc) and
    the kernel trace that goes with them: every kernel family a few times, each
    preceded by enough untimed work of its own to be at its steady clocks.
      1. a plain f32 copy of known size (the calibration kernel: 256 MiB read,
         256 MiB written per dispatch), then the read-only streaming kernel over
         1 GiB (xor_checksum_kernel: the read bandwidth this box sustains)
      2. the decode step (gemv_list_kernel, one dispatch per step), then the
         Gemma-3-1B FFN + vocabulary step (the instantiation with the column tails)
      3. the seven Qwen3-0.6B projections at M = 512 as one group over sealed
         weights (split_act_list_kernel + gemm_bf16x3_kernel, 128-token tiles)
      4. the same over raw weights (gemm_mma kernels, f32 matrix cores)
      5. the Gemma-3-1B vocabulary projection at M = 512 (gemm_bf16x3_kernel)
      6. 2B-class shapes, int8-activation profile at M = 512
         (quantize_act_kernel + gemm_i8_lds_kernel), 8 copies of each matrix, through
         the bit-exact entry point and then through the one with the fused tail
    Prints the algorithmic bytes / operations of each so that the counter values
    per dispatch can be set beside them."""
    n = 64 << 20  # f32 elements
    src, dst = ctx.buffer(n * 4), ctx.buffer(n * 4)
    for _ in range(3):
        ctx.copy_f32(src, 0, dst, 0, n)
    ctx.fence()
    src.free()
    dst.free()
    report = {"copy_f32_kernel": {"read_bytes": n * 4, "written_bytes": n * 4, "dispatches": 3}}
    # 1b. the read-only streaming kernel over 1 GiB (the measured read ceiling)
    report["xor_checksum_kernel"] = read_ceiling(ctx, gib=1, reps=10)
    products, keep, _ = build_decode_step(ctx, keep_host=False)
    step_bytes = sum(S.gemv_bytes(pr.rows, pr.cols) for pr in products)
    run_steps(host, ctx, products, 0, 5, grouped=True)
    report["gemv_list_kernel"] = {
        "algorithmic_bytes_per_dispatch": step_bytes, "timed_dispatches": 5,
        "weights_bytes": sum(S.q8_0_bytes(p.rows, p.cols) for p in products)}
    for obj in keep:
        (obj.buf if isinstance(obj, H.Matrix) else obj).free()
    # 2b. the Gemma-3-1B step (79 GEMVs: rows of 1152 and of 6912 columns), one dispatch per step
    gp, gkeep = [], []
    for c in range(26):
        for name, rows, cols in [s for s in S.GEMMA3_1B if s[0] != "lm_head"]:
            gkeep.append(H.Matrix.load(ctx, S.make_weights(rows, cols, 3000 + 17 * c + len(gp)), cols, rows))
            gp.append((gkeep[-1], rows, cols))
    rows, cols = [s for s in S.GEMMA3_1B if s[0] == "lm_head"][0][1:]
    gkeep.append(H.Matrix.load(ctx, S.make_weights(rows, cols, 3999), cols, rows))
    gp.append((gkeep[-1], rows, cols))
    gprods = []
    for m, rows, cols in gp:
        xb, yb = ctx.buffer(cols * 4), ctx.buffer(rows * 4)
        xb.upload(0, S.make_activations(cols, rows))
        gkeep += [xb, yb]
        gprods.append(tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, 1, TMH_GEMV))
    run_steps(host, ctx, gprods, 0, 5, grouped=True)
    report["gemv_list_kernel, Gemma-3-1B step"] = {
        "algorithmic_bytes_per_dispatch": sum(S.gemv_bytes(p.rows, p.cols) for p in gprods),
        "timed_dispatches": 5, "weights_bytes": sum(S.q8_0_bytes(p.rows, p.cols) for p in gprods)}
    for obj in gkeep:
        (obj.buf if isinstance(obj, H.Matrix) else obj).free()
    M = 512
    for label, seal in (("gemm_bf16x3_kernel, seven projections, sealed", True),
                        ("gemm_mma kernels (f32), seven projections, raw", False)):
        prods, keep = [], []
        for name, rows, cols in S.QWEN3_0_6B_LAYER:
            m = H.Matrix.load(ctx, S.make_weights(rows, cols, S.tensor_seed(2, 0, name)), cols, rows,
                              seal=seal)
            xb, yb = ctx.buffer(M * cols * 4), ctx.buffer(M * rows * 4)
            xb.upload(0, S.make_activations(M * cols, rows))
            keep += [m.buf, xb, yb]
            prods.append(tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, M, TMH_GEMM_MMA))
        run_steps(host, ctx, prods, 0, 5, grouped=True)
        report[label] = {"flops_per_group": sum(2.0 * M * p.rows * p.cols for p in prods),
                         "timed_groups": 5}
        for b in keep:
            b.free()
    rows, cols = [s for s in S.GEMMA3_1B if s[0] == "lm_head"][0][1:]
    m = H.Matrix.load(ctx, S.make_weights(rows, cols, 3999), cols, rows)
    xb, yb = ctx.buffer(M * cols * 4), ctx.buffer(M * rows * 4)
    xb.upload(0, S.make_activations(M * cols, 7))
    run_steps(host, ctx, [tmh_product(m.buf.raw, xb.raw, yb.raw, rows, cols, M, TMH_GEMM_MMA)], 0, 5,
              grouped=False)
    report["gemm_bf16x3_kernel, Gemma lm_head"] = {"flops_per_dispatch": 2.0 * M * rows * cols,
                                                   "timed_dispatches": 5}
    for b in (m.buf, xb, yb):
        b.free()
    pool = _weights_pool(ctx, list(S.SWEEP_2B), 8, 4000)
    widths = sorted({c for _, _, c, _ in pool})
    xb = ctx.buffer(M * max(widths) * 4)
    xb.upload(0, S.make_activations(M * max(widths), 99))
    xqs = {c: ctx.buffer(H.xq_bytes(c, M)) for c in widths}
    ys = [ctx.buffer(M * r * 4) for _, r, _, _ in pool]
    for label, kind in (("gemm_i8_lds_kernel, 2B shapes", TMH_GEMM_I8),
                        ("gemm_i8_lds_kernel with the fused tail, 2B shapes", TMH_GEMM_I8_FMA)):
        prods = [tmh_product(None, xb.raw, xqs[c].raw, 1, c, M, TMH_QUANT) for c in widths]
        prods += [tmh_product(m.buf.raw, xqs[c].raw, yb.raw, r, c, M, kind)
                  for (_, r, c, m), yb in zip(pool, ys)]
        run_steps(host, ctx, prods, 0, 5, grouped=True)
        report[label] = {
            "int8_ops_per_group": sum(2.0 * M * r * c for _, r, c, _ in pool), "timed_groups": 5,
            "products_per_group": len(pool)}
    print(json.dumps(report), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="budget of the CPU-baseline leg (0 skips it)")
    ap.add_argument("--no-gemm", action="store_true",
                    help="decode workload: leave out roofline.gemm_m512 (BASELINE config 2)")
    ap.add_argument("--no-configs", action="store_true",
                    help="decode workload: leave out roofline.gemma and roofline.sweep_2b "
                         "(BASELINE configs 3 and 4)")
    ap.add_argument("--no-recorded", action="store_true",
                    help="chain workload: leave out the recorded-step leg (rocprofv3's kernel trace "
                         "crashed on stream capture here)")
    ap.add_argument("--ungrouped", action="store_true",
                    help="one commit per GEMV instead of one group per step")
    ap.add_argument("--model", choices=sorted(CHAIN_MODELS), default="qwen",
                    help="chain workload: whose shapes the dependent decode step has")
    ap.add_argument("--tokens", type=int, default=1, choices=range(1, 33), metavar="1..32",
                    help="chain workload: tokens per step (more than one: the exact small-batch "
                         "GEMM, as a speculative step verifies its draft)")
    ap.add_argument("--unsealed", action="store_true",
                    help="decode workload: leave the weights in the layout they are uploaded in "
                         "(what a binding that never calls tm_hip_q8_0_pack runs on)")
    ap.add_argument("--workload", choices=["decode", "gemm", "gemma", "sweep", "chain", "f16", "layer",
                                           "traffic"],
                    default="decode",
                    help="decode (default, the headline line, which carries every BASELINE "
                         "configuration); gemm / gemma / sweep print configs 2 / 3 / 4 on their own, "
                         "the sweep with every batch")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one MI355X: this path runs on a single GPU "
                         "(run with --gpus 1)")
    p = H.probe()
    if not p.available:
        raise SystemExit(f"bench.py needs an MI355X: {p.info}")
    host = load_host()
    ctx = H.HipContext.open()
    if args.workload == "traffic":
        run_traffic(host, ctx)
        ctx.close()
        return
    if args.workload != "decode":
        fn = {"gemma": bench_gemma, "sweep": bench_sweep, "chain": bench_chain,
              "f16": bench_f16, "layer": bench_layer, "gemm": bench_gemm}[args.workload]
        extra = ({"recorded": not args.no_recorded, "model": args.model, "tokens": args.tokens}
                 if args.workload == "chain" else {})
        res = fn(host, ctx, args.steps, args.warmup, **extra)
        if isinstance(res, tuple):  # (roofline entry, CPU sample)
            res = {"roofline": res[0], "cpu_baseline": res[1]}
        print(json.dumps(res), flush=True)
        ctx.close()
        return

    ceiling = read_ceiling(ctx)
    products, keep, host_side = build_decode_step(ctx, keep_host=args.cpu_seconds > 0,
                                                  seal=not args.unsealed)
    step_bytes = sum(S.gemv_bytes(pr.rows, pr.cols) for pr in products)
    ctx.fence()
    t = run_steps(host, ctx, products, args.warmup, args.steps, grouped=not args.ungrouped)
    pre = run_steps.last_precondition
    ms_per_step = t.wall_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    launches_per_step = t.launches / args.steps
    launch_us = t.gpu_ms * 1e3 / t.launches
    launch_bytes = step_bytes / launches_per_step
    achieved = launch_bytes / (launch_us * 1e-6) / 1e9
    stats = step_stats(t, args.steps)
    median_launch_us = stats.get("median_us", 0.0) / launches_per_step

    line = {
        "metric": "Q8_0 GEMV achieved HBM GB/s (% peak); Q8_0 GEMM TFLOP/s at M=512",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {
            "workload": "Qwen3-0.6B-shaped decode step at M=1: 28 x {q,k,v,o,gate,up,down} + "
                        "lm_head = 197 Q8_0 GEMVs, f32 activations (BASELINE config 1)",
            "weights_bytes": sum(S.q8_0_bytes(pr.rows, pr.cols) for pr in products),
            "algorithmic_bytes_per_step": step_bytes,
            "issue": "one commit per GEMV" if args.ungrouped else "one dispatch group per step",
            "weights_layout": "as uploaded (34-byte blocks)" if args.unsealed else "sealed",
            "host_issue_us_per_step": t.host_ms * 1e3 / args.steps,
            "pct_of_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
            "precondition": dict(pre, rule="untimed windows of steps until three in a row agree "
                                 "within 1 % on GPU time per step; then --warmup, then --steps"),
            "other_configs": "roofline.gemm_m512 (config 2), roofline.gemma (config 3), "
                             "roofline.sweep_2b (config 4); their CPU samples under "
                             "cpu_baseline.per_config",
        },
        "roofline": {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": (DECODE_STEP_TRAFFIC_BYTES
                        if launches_per_step == 1.0 and not args.unsealed else None),
            "traffic_source": DECODE_STEP_TRAFFIC_SOURCE,
            "kernel": "q8::gemv_list_kernel",
            "launches_per_step": launches_per_step,
            "avg_launch_us": launch_us,
            "median_launch_us": median_launch_us,
            "achieved_at_median": (launch_bytes / (median_launch_us * 1e-6) / 1e9
                                   if median_launch_us > 0 else None),
            "frac_at_median": (launch_bytes / (median_launch_us * 1e-6) / 1e9 / HBM_PEAK_GBS
                               if median_launch_us > 0 else None),
            "step_us": stats,
            "algorithmic_bytes_per_launch": launch_bytes,
            "measured_read_ceiling": ceiling,
            "frac_of_measured_ceiling": achieved / ceiling["gbs"],
        },
    }
    per_config = {}
    if args.cpu_seconds > 0:
        line["cpu_baseline"] = cpu_baseline(host_side, args.cpu_seconds)
        line["cpu_baseline"]["per_config"] = per_config
    for obj in keep:
        (obj.buf if isinstance(obj, H.Matrix) else obj).free()
    host_side = None
    cpu = args.cpu_seconds > 0
    if not args.no_gemm:
        # (the other configurations' legs last milliseconds: they take enough steps for
        # stable means whatever --steps says)
        line["roofline"]["gemm_m512"], per_config["config2_gemm_m512"] = bench_gemm(
            host, ctx, max(100, args.steps // 4), max(10, args.warmup // 4), cpu=cpu)
    if not args.no_configs:
        line["roofline"]["gemma"], per_config["config3_gemma"] = bench_gemma(
            host, ctx, max(100, args.steps // 4), max(10, args.warmup // 4), cpu=cpu)
        line["roofline"]["sweep_2b"], per_config["config4_sweep_2b"] = bench_sweep(
            host, ctx, max(40, args.steps // 4), 0, cpu=cpu, batches=SWEEP_HEADLINE_M + (16, 32, 128))
    ctx.close()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
