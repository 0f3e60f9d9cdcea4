#!/usr/bin/env python3
"""Benchmark of the 8-bit hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

A "step" is one launch of the headline kernel on resident synthetic data: the fp8 e4m3 GEMM with fused
per-token / per-channel dequantisation + bias + tanh-GELU at M=6144, N=8192, K=2048 (bf16 output).
After W warm-up steps exactly K steps are timed between two device synchronisations; the one JSON line
printed at the end carries that throughput as `value` (TFLOP/s), the roofline of the kernel measured with
HIP events on the launch stream, a CPU baseline (the oracle's own float64 function for this workload timed on the
host cores at full size, 25 s budget; a plain fp32 BLAS formulation is reported beside it in `extras`, labelled as
not the oracle), and in `extras` the other workloads of the metric: fp8 Hadamard self-attention
(S=6144, D=64), cross-attention with a padding mask, the int8 GEMM, the memory-bound row kernels and the
DiT block in milliseconds.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 / int8 MFMA, published (no sparsity)
HBM_PEAK_GBS = 8000.0
E4M3 = torch.float8_e4m3fn


def _ramp_clocks(fn, seconds=0.4):
    """Untimed: keep the device busy with `fn` until it has left its idle clock state (the engine clock of an idle
    MI355X takes on the order of 100 ms of load to come up; short timings taken before that read about 25 % low)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def _time(fn, steps, warmup, ramp=0.15):
    """Mean seconds per call over exactly `steps` calls (HIP events on the current stream, which is the
    stream the library launches on). `ramp` seconds of untimed calls come first: every workload here is set up
    on the host while the device idles, and `warmup` calls of a 20-100 us kernel are far shorter than the time
    the engine clock needs to come back up."""
    if ramp > 0:
        _ramp_clocks(fn, ramp)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return start.elapsed_time(stop) * 1e-3 / steps, wall


def _time_cold(make, copies, steps, warmup):
    """Like _time, with every call on a buffer set of its own: make(i) returns the call on the i-th copy of the inputs, the
    results of the last `copies` calls stay allocated (so the allocator hands out other memory for the next ones), and the
    calls go round the copies. With the copies adding up to several times the L2s (8 x 4 MB) and the memory-side cache
    (256 MB), no call finds any of its data left behind by an earlier one: the time of a pass through HBM proper."""
    fns = [make(i) for i in range(copies)]
    ring, pos = [None] * copies, [0]

    def fn():
        i = pos[0] % copies
        ring[i] = fns[i]()
        pos[0] += 1
    t, _ = _time(fn, steps, warmup)
    del ring, fns
    return t


def _gemm_inputs(dev, m, n, k, seed=0):
    from q8_kernels_amd import _C
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16).float()
    xq, sx = _C.tokenwise_quant(x.to(dev), E4M3)
    wq, sw = _C.tokenwise_quant(w.to(dev), E4M3)
    return x, w, bias, xq, sx, wq, sw


def _cpu_baseline_gemm(x, w, bias, budget_s=25.0):
    """The oracle's own fp8 linear + bias + GELU (oracle/q8_oracle.py: ref_quant, then ref_fp8_mm, i.e. e4m3 codes decoded
    to float64, float64 accumulation, the reference's dequantisation order, tanh-GELU, bf16 store) on the host cores at
    the full problem size: run again while the next run still fits the budget, median of the runs."""
    from oracle import q8_oracle as O
    threads = torch.get_num_threads()
    xq, sx = O.ref_quant(x, E4M3)
    wq, sw = O.ref_quant(w, E4M3)
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 and (not times or time.perf_counter() - t_start + max(times) < budget_s):
        t0 = time.perf_counter()
        O.ref_fp8_mm(xq, wq, bias, sx, sw, True, torch.bfloat16)
        times.append(time.perf_counter() - t0)
    sec = sorted(times)[len(times) // 2]
    flop = 2.0 * x.shape[0] * w.shape[0] * x.shape[1]
    return {"value": flop / sec / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "the oracle's ref_fp8_mm (float64) on the full %dx%dx%d fp8 linear+bias+GELU, median of %d run(s), %.1f s each"
                      % (x.shape[0], w.shape[0], x.shape[1], len(times), sec)}


def _cpu_baseline_attn(heads=4, S=6144):
    """The oracle's own fp8 Hadamard attention (oracle/q8_oracle.py: ref_flash_attn_func, i.e. FHT + e4m3 casts + float64
    softmax attention with e4m3-rounded probabilities) on `heads` of the 64 (batch, head) pairs of config 3 at full sequence
    length, on the host cores; the heads are independent, so the rate carries over and the full-size time is 64 / heads times
    the measured one."""
    from oracle import q8_oracle as O
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(1, heads, S, 64, generator=g).to(torch.bfloat16) for _ in range(3))
    t0 = time.perf_counter()
    O.ref_flash_attn_func(q, k, v, None, None, True, out_dtype=torch.bfloat16)
    sec = time.perf_counter() - t0
    flop = 4.0 * heads * S * S * 64
    return {"value": flop / sec / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "the oracle's ref_flash_attn_func on %d of the 64 (batch, head) pairs of B2 H32 S%d D64 (one run, %.1f s); "
                      "heads are independent: the full configuration extrapolates to %.0f s" % (heads, S, sec, sec * 64 / heads),
            "full_size_seconds_extrapolated": sec * 64 / heads}


def _cpu_blas_gemm(x, w, bias):
    """Not the oracle: the same linear + bias + GELU as plain fp32 BLAS on the dequantised codes (torch.matmul on the host
    cores), the fastest CPU formulation at hand, reported beside the oracle's figure for scale."""
    from oracle import q8_oracle as O
    xq, sx = O.ref_quant(x, E4M3)
    wq, sw = O.ref_quant(w, E4M3)

    def run():
        acc = xq.to(torch.float32) @ wq.to(torch.float32).T
        v = acc * (sx[:, None] * sw[None, :]) + bias
        return torch.nn.functional.gelu(v, approximate="tanh").to(torch.bfloat16)

    run()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    sec = sorted(times)[1]
    flop = 2.0 * x.shape[0] * w.shape[0] * x.shape[1]
    return {"tflops": flop / sec / 1e12, "ms": sec * 1e3, "cores": torch.get_num_threads(),
            "what": "fp32 torch.matmul on dequantised e4m3 codes + bias + tanh-GELU -> bf16, full size; not the oracle"}


def _attn_inputs(dev, g, B=2, H=32, S=6144, outliers=True):
    """Q, K, V ~ N(0,1) in bf16; with `outliers` one of the 64 head-dim channels of each tensor (1 %, rounded up; seeded
    choice) is scaled x 20, the inputs BASELINE config 3 names. Returns the per-token quantized operands (Hadamard-rotated
    Q and K) and the reference-style direct casts."""
    from q8_kernels_amd import _C
    q, k, v = (torch.randn(B, H, S, 64, generator=g).to(torch.bfloat16) for _ in range(3))
    if outliers:
        for t in (q, k, v):
            t[..., int(torch.randperm(64, generator=g)[0])] *= 20
    q, k, v = q.to(dev), k.to(dev), v.to(dev)
    qr, kr = _C.fast_hadamard_transform(q, 0.125, torch.bfloat16), _C.fast_hadamard_transform(k, 0.125, torch.bfloat16)
    (q8, sq), (k8, sk), (v8, sv) = _C.tokenwise_quant(qr, E4M3), _C.tokenwise_quant(kr, E4M3), _C.tokenwise_quant(v, E4M3)
    vt = v8.view(torch.uint8).transpose(2, 3).contiguous().view(E4M3)
    s = (1 / 64) ** 0.5 * (0.125 ** 0.5)
    qd, kd = _C.fast_hadamard_transform(q, s, E4M3), _C.fast_hadamard_transform(k, s, E4M3)
    return {"scaled": (q8, k8, vt, sq, sk, sv), "direct": (qd, kd, vt), "fold": s}


def _extras_attn(dev, steps, warmup, g, out):
    """fp8 self-attention with Hadamard at S = 6144 on the inputs of config 3 (one outlier channel x 20 per tensor): per-token
    e4m3 (config 3) and reference-style direct casts; the
    cross-attention with a padding mask (config 4). Each entry carries the quantities a roofline needs: flop, the number
    of exponentials (one per score; the kernel is bound by them), average launch time."""
    from q8_kernels_amd import _C
    B, H, S = 2, 32, 6144
    a = _attn_inputs(dev, g, B, H, S)
    q8, k8, vt, sq, sk, sv = a["scaled"]
    qd, kd, _ = a["direct"]
    flop = 4.0 * B * H * S * S * 64

    def entry(t, kernel):
        return {"ms": t * 1e3, "tflops": flop / t / 1e12, "frac_of_fp8_peak": flop / t / 1e12 / FP8_PEAK_TFLOPS, "shape": "B2 H32 S6144 D64",
                "roofline": {"bound": "mfma", "achieved": flop / t / 1e12, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": flop / t / 1e12 / FP8_PEAK_TFLOPS, "kernel": kernel, "flop_per_launch": flop,
                             "exp2_per_launch": float(B * H) * S * S, "avg_launch_us": t * 1e6}}

    t, _ = _time(lambda: _C.flash_attention(q8, k8, vt, 0.125, None, out_dtype=torch.bfloat16, q_scales=sq, k_scales=sk,
                                            v_scales=sv), steps, warmup)
    out["attn_self_fp8_per_token_scales"] = entry(t, "attn_fwd_kernel<bf16, per-token scales, 4 waves x 32 queries>")
    t, _ = _time(lambda: _C.flash_attention(qd, kd, vt, 1.0, None, out_dtype=torch.bfloat16), steps, warmup)
    out["attn_self_fp8_reference_casts"] = entry(t, "attn_fwd_kernel<bf16, unit scales, 8 waves x 32 queries>")
    # the same two launches on plain N(0,1) inputs without the outlier channel (flat softmax rows: the running maximum moves
    # more often than on the peaked rows the outliers make)
    pl = _attn_inputs(dev, g, B, H, S, outliers=False)
    p8, pk8, pvt, psq, psk, psv = pl["scaled"]
    pqd, pkd, _ = pl["direct"]
    t, _ = _time(lambda: _C.flash_attention(p8, pk8, pvt, 0.125, None, out_dtype=torch.bfloat16, q_scales=psq, k_scales=psk,
                                            v_scales=psv), steps, warmup)
    out["attn_self_fp8_per_token_scales_no_outliers"] = entry(t, "attn_fwd_kernel<bf16, per-token scales, 4 waves x 32 queries>")
    t, _ = _time(lambda: _C.flash_attention(pqd, pkd, pvt, 1.0, None, out_dtype=torch.bfloat16), steps, warmup)
    out["attn_self_fp8_reference_casts_no_outliers"] = entry(t, "attn_fwd_kernel<bf16, unit scales, 8 waves x 32 queries>")
    del pl, p8, pk8, pvt, psq, psk, psv, pqd, pkd
    v_tok = vt.view(torch.uint8).transpose(2, 3).contiguous().view(E4M3)  # [B,H,S,64]: V as the fused prologue leaves it
    t, _ = _time(lambda: _C.flash_attention(qd, kd, v_tok, 1.0, None, out_dtype=torch.bfloat16, v_token_major=True), steps, warmup)
    out["attn_self_fp8_reference_casts_token_major_v"] = entry(t, "attn_fwd_kernel<bf16, unit scales, 8 waves x 32 queries, token-major V>")
    # cross-attention with a padding mask (config 4): HBM-bound
    N = 128
    kx, vx = (torch.randn(B, H, N, 64, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    lens = torch.randint(16, 129, (B,), generator=g, dtype=torch.int32).to(dev)
    kx8 = _C.fast_hadamard_transform(kx, a["fold"], E4M3)
    vxt = vx.to(E4M3).view(torch.uint8).transpose(2, 3).contiguous().view(E4M3)
    t, _ = _time(lambda: _C.flash_attention(qd, kx8, vxt, 1.0, lens, out_dtype=torch.bfloat16), steps, warmup)
    (kx8s, skx), (vx8s, svx) = _C.tokenwise_quant(_C.fast_hadamard_transform(kx, 0.125, torch.bfloat16), E4M3), _C.tokenwise_quant(vx, E4M3)
    vxts = vx8s.view(torch.uint8).transpose(2, 3).contiguous().view(E4M3)
    t_scaled, _ = _time(lambda: _C.flash_attention(q8, kx8s, vxts, 0.125, lens, out_dtype=torch.bfloat16, q_scales=sq, k_scales=skx,
                                                   v_scales=svx), steps, warmup)
    byts = B * H * (S * 64 + 2 * N * 64 + S * 64 * 2)
    out["attn_cross_fp8_masked"] = {"ms": t * 1e3, "gbs": byts / t / 1e9, "frac_of_hbm_peak": byts / t / 1e9 / HBM_PEAK_GBS,
                                    "tflops": 4.0 * B * H * S * N * 64 / t / 1e12, "shape": "B2 H32 Sq6144 Skv128 D64",
                                    "valid_lengths": lens.tolist(), "kernel": "attn_short_kernel<bf16>"}
    byts_s = byts + B * H * (S + 2 * N) * 4  # the per-token scales as well
    out["attn_cross_fp8_masked_per_token_scales"] = {
        "ms": t_scaled * 1e3, "gbs": byts_s / t_scaled / 1e9, "frac_of_hbm_peak": byts_s / t_scaled / 1e9 / HBM_PEAK_GBS,
        "tflops": 4.0 * B * H * S * N * 64 / t_scaled / 1e12, "shape": "B2 H32 Sq6144 Skv128 D64", "valid_lengths": lens.tolist(),
        "kernel": "attn_short_kernel<bf16, per-token scales>"}


def _extras_gemm(dev, steps, warmup, g, out):
    from q8_kernels_amd import _C
    # int8 GEMM (config 2)
    # (operands as config 2 defines them: symmetric per-row int8 quantisation, round half even, of N(0,1) and N(0,0.02))
    a, sa = _C.tokenwise_quant(torch.randn(6144, 2048, generator=g).to(torch.bfloat16).to(dev), None, round_half_even=True)
    b, sb = _C.tokenwise_quant((torch.randn(2048, 2048, generator=g) * 0.02).to(torch.bfloat16).to(dev), None, round_half_even=True)
    bias = (torch.randn(2048, generator=g) * 0.02).to(dev)
    t, _ = _time(lambda: _C.q8_mm_bias(a, b, bias, sa, sb, False, torch.bfloat16), steps, warmup)
    ops = 2.0 * 6144 * 2048 * 2048
    out["int8_gemm_6144x2048x2048"] = {"ms": t * 1e3, "tops": ops / t / 1e12,
                                       "roofline": {"bound": "mfma", "achieved": ops / t / 1e12, "peak": FP8_PEAK_TFLOPS, "unit": "TOP/s",
                                                    "frac": ops / t / 1e12 / FP8_PEAK_TFLOPS, "kernel": "gemm_persist_kernel<int8>",
                                                    "ops_per_launch": ops, "avg_launch_us": t * 1e6}}
    # the fp8 linear as the reference's FP8LinearFunc runs it (q8_kernels/functional/linear.py:138-159): the bf16 activation is
    # quantized inside the call, the weight arrives quantized; with and without the fused GELU of the FFN's first layer
    from q8_kernels_amd.functional.linear import fp8_linear
    xb, _, lb, _, _, lwq, lsw = _gemm_inputs(dev, 6144, 8192, 2048)
    xb, lb = xb.to(dev), lb.to(dev)
    lflop = 2.0 * 6144 * 8192 * 2048
    for name, gelu in (("fp8_linear_quant_plus_gemm_6144x8192x2048", False), ("fp8_linear_quant_plus_gemm_gelu_6144x8192x2048", True)):
        t, _ = _time(lambda: fp8_linear(xb, lwq, lb, None, lsw, False, torch.bfloat16, fuse_gelu=gelu), steps, warmup)
        out[name] = {"ms": t * 1e3, "tflops": lflop / t / 1e12, "frac_of_fp8_peak": lflop / t / 1e12 / FP8_PEAK_TFLOPS,
                     "what": "bf16 [6144,2048] in -> per-token e4m3 quantizer -> GEMM + bias%s -> bf16; effective rate of the two launches" % (" + GELU" if gelu else "")}
    tq, _ = _time(lambda: _C.tokenwise_quant(xb, E4M3), steps, warmup)
    out["fp8_linear_quant_plus_gemm_6144x8192x2048"]["quantizer_alone_ms"] = tq * 1e3
    del xb, lwq
    # fp8 GEMMs of the block without GELU: projection (K = 2048) and FFN down projection (K = 8192), M = 12288 tokens
    for name, (mm, nn, kk) in (("fp8_gemm_12288x2048x2048", (12288, 2048, 2048)), ("fp8_gemm_12288x2048x8192", (12288, 2048, 8192))):
        _, _, gb, gxq, gsx, gwq, gsw = _gemm_inputs(dev, mm, nn, kk, seed=2)
        gb = gb.to(dev)
        t, _ = _time(lambda: _C.fp8_mm_bias(gxq, gwq, gb, gsx, gsw, False, torch.bfloat16), steps, warmup)
        out[name] = {"ms": t * 1e3, "tflops": 2.0 * mm * nn * kk / t / 1e12, "frac_of_fp8_peak": 2.0 * mm * nn * kk / t / 1e12 / FP8_PEAK_TFLOPS}
        if kk == 2048:
            # the reference's default output type: out_type None -> e4m3 (csrc/gemm/q8_gemm_api.cpp:82-87), fp8 and int8 operands
            t, _ = _time(lambda: _C.fp8_mm_bias(gxq, gwq, gb, gsx, gsw, False, None), steps, warmup)
            out[name + "_e4m3_out"] = {"ms": t * 1e3, "tflops": 2.0 * mm * nn * kk / t / 1e12,
                                       "frac_of_fp8_peak": 2.0 * mm * nn * kk / t / 1e12 / FP8_PEAK_TFLOPS}
            ai, bi = gxq.view(torch.int8), gwq.view(torch.int8)  # any int8 codes do for timing
            t, _ = _time(lambda: _C.q8_mm_bias(ai, bi, gb, gsx, gsw, False, None), steps, warmup)
            out["int8_gemm_%dx%dx%d_e4m3_out" % (mm, nn, kk)] = {"ms": t * 1e3, "tops": 2.0 * mm * nn * kk / t / 1e12}
        del gxq, gwq


def _time_replay(fn, calls=50, replays=4):
    """Mean seconds per call of `fn` captured `calls` times into one HIP graph and replayed: for kernels that take less
    time than a call's host side (a few microseconds), where back-to-back eager calls would time the host."""
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    graph, stream = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(3):
            fn()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(calls):
                fn()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / (replays * calls)


def _extras_gemm_small(dev, steps, warmup, g, out):
    """The shapes beside the big projections: the K / V projection of the 256 text rows (small-problem kernel, 64x64 tiles),
    a 2048-cube (128x128 tiles), and the QKV projection with the cast of V in its epilogue next to the plain GEMM."""
    from q8_kernels_amd import _C
    for mm, nn, kk in ((256, 4096, 2048), (2048, 2048, 2048)):
        _, _, gb, gxq, gsx, gwq, gsw = _gemm_inputs(dev, mm, nn, kk, seed=4)
        gb = gb.to(dev)
        t = _time_replay(lambda: _C.fp8_mm_bias(gxq, gwq, gb, gsx, gsw, False, torch.bfloat16))
        out["fp8_gemm_%dx%dx%d_graph_replay" % (mm, nn, kk)] = {"ms": t * 1e3, "tflops": 2.0 * mm * nn * kk / t / 1e12}
    mm, nn, kk = 12288, 6144, 2048
    _, _, gb, gxq, gsx, gwq, gsw = _gemm_inputs(dev, mm, nn, kk, seed=5)
    gb = gb.to(dev)
    t, _ = _time(lambda: _C.fp8_mm_bias(gxq, gwq, gb, gsx, gsw, False, torch.bfloat16), steps, warmup)
    out["fp8_gemm_qkv_12288x6144x2048"] = {"ms": t * 1e3, "tflops": 2.0 * mm * nn * kk / t / 1e12,
                                          "frac_of_fp8_peak": 2.0 * mm * nn * kk / t / 1e12 / FP8_PEAK_TFLOPS}
    t, _ = _time(lambda: _C.mm_bias_qkv(gxq, gwq, gb, gsx, gsw, 6144, 4096), steps, warmup)
    out["fp8_gemm_qkv_12288x6144x2048_v_cast_in_epilogue"] = {"ms": t * 1e3, "tflops": 2.0 * mm * nn * kk / t / 1e12,
                                                             "frac_of_fp8_peak": 2.0 * mm * nn * kk / t / 1e12 / FP8_PEAK_TFLOPS}


def _extras_library(dev, steps, warmup, g, out):
    """Yardstick, not product: the vendor library's fp8 GEMM (hipBLASLt through torch._scaled_mm, row-wise scales, bf16
    output, no bias, no activation) on the same operands, box and process as this repository's kernel with its fused
    bias (+ GELU) epilogue."""
    from q8_kernels_amd import _C
    for (mm, nn, kk) in ((6144, 8192, 2048), (8192, 8192, 8192), (12288, 2048, 8192), (12288, 2048, 2048)):
        _, _, gb, gxq, gsx, gwq, gsw = _gemm_inputs(dev, mm, nn, kk, seed=3)
        gb = gb.to(dev)
        flop = 2.0 * mm * nn * kk
        entry = {}
        try:
            sa2, sb2, wt = gsx.view(-1, 1), gsw.view(1, -1), gwq.t()
            t, _ = _time(lambda: torch._scaled_mm(gxq, wt, scale_a=sa2, scale_b=sb2, out_dtype=torch.bfloat16), steps, warmup)
            entry["library_scaled_mm"] = {"ms": t * 1e3, "frac_of_fp8_peak": flop / t / 1e12 / FP8_PEAK_TFLOPS}
        except Exception as e:  # the yardstick is optional: an unsupported call must not take the bench line down
            entry["library_scaled_mm"] = {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}
        for name, gelu in (("this_kernel_bias", False), ("this_kernel_bias_gelu", True)):
            t, _ = _time(lambda: _C.fp8_mm_bias(gxq, gwq, gb, gsx, gsw, gelu, torch.bfloat16), steps, warmup)
            entry[name] = {"ms": t * 1e3, "frac_of_fp8_peak": flop / t / 1e12 / FP8_PEAK_TFLOPS}
        out["library_yardstick_fp8_gemm_%dx%dx%d" % (mm, nn, kk)] = entry
        del gxq, gwq
    # attention: the library's bf16 flash attention (torch scaled_dot_product_attention) at the shape of config 3, next to
    # this repository's fp8 kernel on Hadamard-rotated e4m3 operands (direct casts and per-token scales)
    B, H, S = 2, 32, 6144
    flop = 4.0 * B * H * S * S * 64
    a = _attn_inputs(dev, g, B, H, S)
    q8, k8, vt, sq, sk, sv = a["scaled"]
    qd, kd, _ = a["direct"]
    entry = {}
    try:
        qb, kb, vb = (torch.randn(B, H, S, 64, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
        t, _ = _time(lambda: torch.nn.functional.scaled_dot_product_attention(qb, kb, vb), steps, warmup)
        entry["library_sdpa_bf16"] = {"ms": t * 1e3, "tflops": flop / t / 1e12}
        del qb, kb, vb
    except Exception as e:
        entry["library_sdpa_bf16"] = {"error": "%s: %s" % (type(e).__name__, str(e)[:200])}
    t, _ = _time(lambda: _C.flash_attention(qd, kd, vt, 1.0, None, out_dtype=torch.bfloat16), steps, warmup)
    entry["this_kernel_fp8_direct_casts"] = {"ms": t * 1e3, "tflops": flop / t / 1e12}
    t, _ = _time(lambda: _C.flash_attention(q8, k8, vt, 0.125, None, out_dtype=torch.bfloat16, q_scales=sq, k_scales=sk,
                                            v_scales=sv), steps, warmup)
    entry["this_kernel_fp8_per_token_scales"] = {"ms": t * 1e3, "tflops": flop / t / 1e12}
    out["library_yardstick_attention_B2_H32_S6144_D64"] = entry


def _extras_rows(dev, steps, warmup, g, out):
    from q8_kernels_amd import _C
    # row kernels on [12288, 2048] tokens
    x = torch.randn(12288, 2048, generator=g).to(torch.bfloat16).to(dev)
    n = x.numel()
    cos, sin = torch.randn(12288, 2048, generator=g).to(dev), torch.randn(12288, 2048, generator=g).to(dev)
    w = torch.ones(2048, device=dev)
    for name, fn, bpe in (("quant_fp8", lambda: _C.tokenwise_quant(x, E4M3), 3), ("quant_int8", lambda: _C.tokenwise_quant(x, None), 3),
                          ("fht_bf16", lambda: _C.fast_hadamard_transform(x, 2048 ** -0.5, None), 4),
                          ("rmsnorm_bf16", lambda: _C.rms_norm(x, w, None), 4), ("rope_bf16", lambda: _C.rope(x, cos, sin, None), 12)):
        t, _ = _time(fn, steps, warmup)
        out[name] = {"ms": t * 1e3, "gbs": n * bpe / t / 1e9, "frac_of_hbm_peak": n * bpe / t / 1e9 / HBM_PEAK_GBS}
    # fused row kernels: FHT + int8 quantizer, RMSNorm + e4m3 quantizer (2 B in, 1 B out per element), and the attention
    # prologue RoPE + head split + FHT-64 + e4m3 cast (2 B in + 8 B of tables, 1 B out)
    xs = x.view(2, 6144, 2048)
    cs3, sn3 = cos.view(2, 6144, 2048), sin.view(2, 6144, 2048)
    for name, fn, bpe in (("fht_quant_int8_fused", lambda: _C.fht_quant(x, 2048 ** -0.5, None), 3),
                          ("rmsnorm_quant_fp8_fused", lambda: _C.rms_norm_quant(x, w, E4M3), 3),
                          ("attn_prep_qk_rope_fht_fp8", lambda: _C.attn_prep_qk(xs, 32, cs3, sn3, True, 0.125), 11),
                          ("attn_prep_v_fp8", lambda: _C.attn_prep_v(xs, 32), 3),
                          # Q, K, V of a self-attention in one pass: 3 x 2 B in, 8 B of tables (read once), 3 x 1 B out
                          ("attn_prep_qkv_rope_fht_fp8", lambda: _C.attn_prep_qkv(xs, xs, xs, 32, cs3, sn3, True, 0.125), 17)):
        t, _ = _time(fn, steps, warmup)
        out[name] = {"ms": t * 1e3, "gbs": n * bpe / t / 1e9, "frac_of_hbm_peak": n * bpe / t / 1e9 / HBM_PEAK_GBS}
    # the paired prologue of a self-attention (Q and K) on the tables as the model builds them - every angle twice, one
    # position grid for the batch - in full [2, 6144, 2048] (2 x 2 B in, 8 B of tables, 2 x 1 B out per element) and
    # with the repeated values stored once ([1, 6144, 1024]: 1 B of tables per element), as the modules pass them
    ang = torch.rand(1, 6144, 1024, generator=g) * 6.28
    cf = torch.cos(ang).repeat_interleave(2, -1).expand(2, -1, -1).contiguous().to(dev)
    sf = torch.sin(ang).repeat_interleave(2, -1).expand(2, -1, -1).contiguous().to(dev)
    ch, sh = torch.cos(ang).to(dev), torch.sin(ang).to(dev)
    for name, fn, bpe in (("attn_prep_qk_pair_rope_fht_fp8", lambda: _C.attn_prep_qk_pair(xs, xs, 32, cf, sf, True, 0.125), 14),
                          ("attn_prep_qk_pair_rope_fht_fp8_compact_tables", lambda: _C.attn_prep_qk_pair(xs, xs, 32, ch, sh, True, 0.125), 7)):
        t, _ = _time(fn, steps, warmup)
        out[name] = {"ms": t * 1e3, "gbs": n * bpe / t / 1e9, "frac_of_hbm_peak": n * bpe / t / 1e9 / HBM_PEAK_GBS}
    del cf, sf, ch, sh, ang
    # the same kernels with nothing left in any cache by the previous call (16 sets of inputs and outputs, 1.2-5 GB)
    copies = 16
    xc = [x.clone() for _ in range(copies)]
    for name, make, bpe in (("quant_fp8", lambda i: (lambda: _C.tokenwise_quant(xc[i], E4M3)), 3),
                            ("quant_int8", lambda i: (lambda: _C.tokenwise_quant(xc[i], None)), 3),
                            ("fht_bf16", lambda i: (lambda: _C.fast_hadamard_transform(xc[i], 2048 ** -0.5, None)), 4),
                            ("rmsnorm_bf16", lambda i: (lambda: _C.rms_norm(xc[i], w, None)), 4),
                            ("fht_quant_int8_fused", lambda i: (lambda: _C.fht_quant(xc[i], 2048 ** -0.5, None)), 3),
                            ("rmsnorm_quant_fp8_fused", lambda i: (lambda: _C.rms_norm_quant(xc[i], w, E4M3)), 3)):
        t = _time_cold(make, copies, steps, warmup)
        out.setdefault(name, {}).update({"ms_cold": t * 1e3, "gbs_cold": n * bpe / t / 1e9, "frac_of_hbm_peak_cold": n * bpe / t / 1e9 / HBM_PEAK_GBS})
    # yardstick: the library's plain copy of the same tensor (2 B in, 2 B out), warm and cold
    t, _ = _time(lambda: x.clone(), steps, warmup)
    out["library_copy_bf16_yardstick"] = {"ms": t * 1e3, "gbs": n * 4 / t / 1e9, "frac_of_hbm_peak": n * 4 / t / 1e9 / HBM_PEAK_GBS}
    t = _time_cold(lambda i: (lambda: xc[i].clone()), copies, steps, warmup)
    out["library_copy_bf16_yardstick"].update({"ms_cold": t * 1e3, "gbs_cold": n * 4 / t / 1e9, "frac_of_hbm_peak_cold": n * 4 / t / 1e9 / HBM_PEAK_GBS})
    cc, sc = [cos.clone() for _ in range(copies)], [sin.clone() for _ in range(copies)]
    for name, make, bpe in (("rope_bf16", lambda i: (lambda: _C.rope(xc[i], cc[i], sc[i], None)), 12),
                            ("attn_prep_qkv_rope_fht_fp8", lambda i: (lambda: _C.attn_prep_qkv(
                                xc[i].view(2, 6144, 2048), xc[(i + 5) % copies].view(2, 6144, 2048), xc[(i + 10) % copies].view(2, 6144, 2048), 32,
                                cc[i].view(2, 6144, 2048), sc[i].view(2, 6144, 2048), True, 0.125)), 17)):
        t = _time_cold(make, copies, steps, warmup)
        out.setdefault(name, {}).update({"ms_cold": t * 1e3, "gbs_cold": n * bpe / t / 1e9, "frac_of_hbm_peak_cold": n * bpe / t / 1e9 / HBM_PEAK_GBS})
    del cc, sc, xc
    del x, cos, sin
    # the Hadamard rotation + int8 quantizer over the 8192-wide FFN hidden of the int8 block
    xw = torch.randn(12288, 8192, generator=g).to(torch.bfloat16).to(dev)
    t, _ = _time(lambda: _C.fht_quant(xw, 8192 ** -0.5, None), steps, warmup)
    out["fht_quant_int8_fused_12288x8192"] = {"ms": t * 1e3, "gbs": xw.numel() * 3 / t / 1e9, "frac_of_hbm_peak": xw.numel() * 3 / t / 1e9 / HBM_PEAK_GBS}


def _graph_replay_time(fn, steps, warmup):
    """fn() captured once into a HIP graph (after two eager calls on the capture stream) and replayed: the block as a pure
    sequence of kernel launches without the host-side work of the Python layer between them."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        keep = fn()
    t, _ = _time(graph.replay, steps, warmup)
    del keep, graph
    return t


class _OpTimer:
    """Stands in for the loaded C-ABI library while one block is profiled: every entry point that launches work is bracketed
    by two HIP events on the launch stream, so that a block comes apart into its operators in call order."""
    # positions of (M, N, K) and of the two batch counts among the entry point's arguments
    _SHAPE_ARGS = {"q8_gemm": ((8, 9, 10), (6, 7)), "q8_gemm_residual": ((9, 10, 11), (7, 8)), "q8_gemm_qkv": ((7, 8, 9), None),
                   "q8_gemm_gated_residual": ((9, 10, 11), None)}

    def __init__(self, handle):
        self._h = handle
        self.calls = []

    def __getattr__(self, name):
        fn = getattr(self._h, name)
        if not name.startswith("q8_") or name in ("q8_strerror", "q8_last_error", "q8_device_info", "q8_gemm_set_config",
                                                  "q8_attn_set_config", "q8_gemm_last_kernel"):
            return fn

        def timed(*args):
            label = name
            if name in self._SHAPE_ARGS:
                mnk, batch = self._SHAPE_ARGS[name]
                label += " %dx%dx%d" % tuple(args[i] for i in mnk)
                if batch is not None and max(args[batch[0]], args[batch[1]]) > 1:
                    label += " x batch %d" % max(args[batch[0]], args[batch[1]])
            elif name == "q8_attn_fwd":
                label += " B%d H%d M%d N%d" % (args[8], args[9], args[10], args[11])
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            r = fn(*args)
            b.record()
            self.calls.append((label, a, b))
            return r
        return timed


def _op_breakdown(fn, block_ms, reps=10):
    """Per-operator times of one call of `fn` (a block): HIP events around every C-ABI entry point, averaged over `reps`
    calls, in call order. `sum_ms` is the sum of the operators' own times, `span_ms` first start to last end (it also holds
    what lies between the operators); `block_ms` is the block timed without the events."""
    from q8_kernels_amd import _lib
    real = _lib.lib()
    timer = _OpTimer(real)
    _ramp_clocks(fn, 0.15)
    _lib._lib = timer
    try:
        runs = []
        for _ in range(reps):
            timer.calls = []
            fn()
            torch.cuda.synchronize()
            runs.append(timer.calls)
    finally:
        _lib._lib = real
    n = len(runs[0])
    assert all(len(r) == n and [c[0] for c in r] == [c[0] for c in runs[0]] for r in runs), "the block's call sequence changed between runs"
    ops = []
    for i in range(n):
        us = sorted(r[i][1].elapsed_time(r[i][2]) * 1e3 for r in runs)[len(runs) // 2]
        ops.append({"op": runs[0][i][0], "us": round(us, 2)})
    span = sorted(r[0][1].elapsed_time(r[-1][2]) for r in runs)[len(runs) // 2]
    total = sum(o["us"] for o in ops) * 1e-3
    return {"ops": ops, "sum_ms": total, "span_ms": span, "block_ms": block_ms, "sum_over_block": total / block_ms,
            "how": "median over %d calls of HIP-event pairs around each C-ABI entry point, in call order; the event records "
                   "themselves sit in the stream (two per operator), which is why the sum reads a few percent above block_ms" % reps}


def _extras_blocks(dev, steps, warmup, g, out):
    from q8_kernels_amd import _C
    from q8_kernels_amd.blocks import Fp8DiTBlock
    from q8_kernels_amd.functional.rope import precompute_freqs_cis, video_index_grid
    # the DiT block (config 5)
    blk = Fp8DiTBlock(device=dev).init_random()
    hidden = torch.randn(2, 6144, 2048, generator=g).to(torch.bfloat16).to(dev)
    text = torch.randn(2, 128, 2048, generator=g).to(torch.bfloat16).to(dev)
    lens = torch.randint(16, 129, (2,), generator=g, dtype=torch.int32).to(dev)
    cosf, sinf = precompute_freqs_cis(video_index_grid(16, 16, 24, batch=2, device=dev), 2048)
    with torch.no_grad():
        t, _ = _time(lambda: blk(hidden, text, (cosf, sinf), lens), max(3, steps // 4), max(1, warmup // 2))
    out["dit_block"] = {"ms": t * 1e3, "gflop": 2079.0, "tflops": 2079.0e9 / t / 1e12, "shape": "tokens [2,6144,2048], text [2,128,2048]"}
    with torch.no_grad():
        t = _graph_replay_time(lambda: blk(hidden, text, (cosf, sinf), lens), max(3, steps // 4), max(1, warmup // 2))
        out["dit_block"]["ms_graph_replay"] = t * 1e3
        out["dit_block"]["breakdown"] = _op_breakdown(lambda: blk(hidden, text, (cosf, sinf), lens), out["dit_block"]["ms"])
    del blk
    # the reference's own block: AdaLN-modulated LTXTransformerBlock on int8 (Hadamard-rotated) Q8Linear layers
    from q8_kernels_amd.blocks import LTXTransformerBlock
    from q8_kernels_amd.modules import Q8Linear
    ltx = LTXTransformerBlock(2048, 32, 64, 2048, bias=True, use_rope=True, norm_affine=False).to(dev)
    for m in ltx.modules():
        if isinstance(m, Q8Linear):
            wq = (torch.randn(m.weight.shape, generator=g) * 0.02).to(torch.bfloat16).to(dev)
            m.weight.data, m.scales.data = _C.fht_quant(wq, wq.shape[-1] ** -0.5, None)
            m.bias.data = (torch.randn(m.bias.shape, generator=g) * 0.02).to(dev)
            del wq
    timestep = (torch.randn(2, 1, 6 * 2048, generator=g) * 0.3).to(dev)
    with torch.no_grad():
        t, _ = _time(lambda: ltx(hidden, (cosf, sinf), None, text, lens, timestep, attn_type="q8_kernels"),
                     max(3, steps // 4), max(1, warmup // 2))
    out["ltx_transformer_block_int8"] = {"ms": t * 1e3, "gflop": 2079.0, "tflops": 2079.0e9 / t / 1e12,
                                         "shape": "tokens [2,6144,2048], text [2,128,2048], int8 linears, fp8 attention"}
    with torch.no_grad():
        t = _graph_replay_time(lambda: ltx(hidden, (cosf, sinf), None, text, lens, timestep, attn_type="q8_kernels"),
                               max(3, steps // 4), max(1, warmup // 2))
        out["ltx_transformer_block_int8"]["ms_graph_replay"] = t * 1e3
        out["ltx_transformer_block_int8"]["breakdown"] = _op_breakdown(
            lambda: ltx(hidden, (cosf, sinf), None, text, lens, timestep, attn_type="q8_kernels"), out["ltx_transformer_block_int8"]["ms"])


def _extras_attn_options(dev, steps, warmup, g, out):
    """The opt-in forms of the self-attention kernel (flags of q8_attn_fwd that change the arithmetic within the stated
    tolerance; off by default and not used by the modules). A group of its own because two of them run the same kernel
    symbols as the default calls: a per-kernel profile of the defaults leaves this group out (--skip attn_options)."""
    from q8_kernels_amd import _C
    B, H, S = 2, 32, 6144
    a = _attn_inputs(dev, g, B, H, S)
    q8, k8, vt, sq, sk, sv = a["scaled"]
    qd, kd, _ = a["direct"]
    flop = 4.0 * B * H * S * S * 64

    def entry(t, kernel):
        return {"ms": t * 1e3, "tflops": flop / t / 1e12, "frac_of_fp8_peak": flop / t / 1e12 / FP8_PEAK_TFLOPS, "shape": "B2 H32 S6144 D64",
                "kernel": kernel}

    # opt-in: the maximum trails the running maximum (fewer rescalings of O; the largest weight of a row is not exact)
    t, _ = _time(lambda: _C.flash_attention(qd, kd, vt, 1.0, None, out_dtype=torch.bfloat16, lazy_max=True), steps, warmup)
    out["attn_self_fp8_reference_casts_lazy_max"] = entry(t, "attn_fwd_kernel<bf16, unit scales, 8 waves x 32 queries>, Q8_ATTN_LAZY_MAX")
    # opt-in: the row sum over the rounded probabilities, taken by the matrix pipe; alone and with the trailing maximum
    t, _ = _time(lambda: _C.flash_attention(qd, kd, vt, 1.0, None, out_dtype=torch.bfloat16, sum_rounded_p=True), steps, warmup)
    out["attn_self_fp8_reference_casts_sum_rounded_p"] = entry(t, "attn_fwd_kernel<bf16, unit scales, 8 waves x 32 queries, row sum by MFMA>")
    t, _ = _time(lambda: _C.flash_attention(qd, kd, vt, 1.0, None, out_dtype=torch.bfloat16, sum_rounded_p=True, lazy_max=True), steps, warmup)
    out["attn_self_fp8_reference_casts_sum_rounded_p_lazy_max"] = entry(t, "attn_fwd_kernel<bf16, unit scales, 8 waves x 32 queries, row sum by MFMA>, Q8_ATTN_LAZY_MAX")
    t, _ = _time(lambda: _C.flash_attention(q8, k8, vt, 0.125, None, out_dtype=torch.bfloat16, q_scales=sq, k_scales=sk, v_scales=sv,
                                            lazy_max=True), steps, warmup)
    out["attn_self_fp8_per_token_scales_lazy_max"] = entry(t, "attn_fwd_kernel<bf16, per-token scales, 4 waves x 32 queries>, Q8_ATTN_LAZY_MAX")


EXTRA_GROUPS = {"attn": _extras_attn, "attn_options": _extras_attn_options, "gemm": _extras_gemm, "gemm_small": _extras_gemm_small, "rows": _extras_rows, "blocks": _extras_blocks,
                "library": _extras_library}


def _extras(dev, steps, warmup, only=None, skip=()):
    """The other workloads of the metric. `only` (group names out of attn, attn_options, gemm, gemm_small, rows, blocks, library) restricts
    the run to those groups, `skip` leaves groups out, e.g. for a counter-collection run of one kernel."""
    out = {}
    for name, fn in EXTRA_GROUPS.items():
        if (only is None or name in only) and name not in skip:
            fn(dev, steps, warmup, torch.Generator().manual_seed(1 + sorted(EXTRA_GROUPS).index(name)), out)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true", help="only the headline GEMM")
    ap.add_argument("--only", default=None,
                    help="comma-separated groups of the other workloads to run (attn, attn_options, gemm, gemm_small, rows, blocks, library)")
    ap.add_argument("--skip", default="", help="comma-separated groups of the other workloads to leave out")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain device copy of 512 MiB (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (nothing on this path communicates "
              "between GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from q8_kernels_amd import _C, _lib
    _lib.lib()  # fail loudly if the HIP library has not been built
    dev = torch.device("cuda:0")
    M, N, K = 6144, 8192, 2048
    x, w, bias, xq, sx, wq, sw = _gemm_inputs(dev, M, N, K)
    bias_d = bias.to(dev)
    step = lambda: _C.fp8_mm_bias(xq, wq, bias_d, sx, sw, True, torch.bfloat16)  # noqa: E731
    if args.copy_calibration:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 512 MiB, writes 512 MiB
        torch.cuda.synchronize()
        del src, dst
    _ramp_clocks(step)
    sec, wall = _time(step, args.steps, args.warmup)
    flop = 2.0 * M * N * K
    tflops = flop / sec / 1e12
    result = {
        "metric": "fp8 GEMM & fp8 attn TFLOPS at LTX shapes, % of gfx950 MFMA peak; block ms",
        "value": tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {"workload": "fp8 e4m3 GEMM + per-token/per-channel dequant + bias + tanh-GELU -> bf16, M=6144 N=8192 K=2048",
                   "inputs": "X~N(0,1), W~N(0,0.02), bias~N(0,0.02), per-row absmax e4m3 quantisation, resident in HBM"},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / FP8_PEAK_TFLOPS,
                     "traffic": None, "kernel": "gemm_persist_kernel<e4m3, gelu>", "flop_per_launch": flop,
                     "avg_launch_us": sec * 1e6, "host_wall_us_per_step": wall * 1e6},
    }
    traffic_file = os.path.join(ROOT, "profiles", "gemm_fp8_traffic.json")
    if os.path.exists(traffic_file):
        # not measured by this run (counters need rocprofv3): the figure of the two --pmc runs summarised under profiles/
        with open(traffic_file) as fh:
            tr = json.load(fh)
        result["roofline"]["traffic"] = tr.get("hbm_bytes_per_launch")
        result["roofline"]["traffic_source"] = tr.get("source")
    if not args.no_cpu:
        result["cpu_baseline"] = _cpu_baseline_gemm(x, w, bias)
    else:
        result["cpu_baseline"] = None
    if not args.no_extras:
        only = None if args.only is None else set(args.only.split(","))
        result["extras"] = _extras(dev, args.steps, args.warmup, only, set(filter(None, args.skip.split(","))))
        # the self-attention of config 3 in its two quantisation modes, each with its own kernel, rate and roofline
        for key, mode in (("attn_self_fp8_per_token_scales", "per_token_scales"), ("attn_self_fp8_reference_casts", "unit_scales")):
            a = result["extras"].get(key)
            if a is not None:
                result["attn_%s_tflops" % mode] = a["tflops"]
                result["attn_%s_frac_of_fp8_peak" % mode] = a["frac_of_fp8_peak"]
                result["attn_%s_roofline" % mode] = a["roofline"]
        if "int8_gemm_6144x2048x2048" in result["extras"]:
            result["int8_gemm_roofline"] = result["extras"]["int8_gemm_6144x2048x2048"]["roofline"]
        if "dit_block" in result["extras"]:
            result["block_ms"] = result["extras"]["dit_block"]["ms"]
        if not args.no_cpu:
            result["extras"]["cpu_fp32_blas_linear_gelu"] = _cpu_blas_gemm(x, w, bias)
            if only is None or "attn" in only:
                result["attn_cpu_baseline"] = _cpu_baseline_attn()
            if "dit_block" in result["extras"] and "attn_cpu_baseline" in result:
                # derived, not run: the block's 1447 GFLOP of GEMMs at the oracle's measured GEMM rate plus its 631 GFLOP of
                # attention at the oracle's measured attention rate (the row operators are negligible beside them)
                sec = 1447.0e9 / (result["cpu_baseline"]["value"] * 1e12) + 631.4e9 / (result["attn_cpu_baseline"]["value"] * 1e12)
                result["block_cpu_baseline"] = {"value": sec * 1e3, "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
                                                "sample": "derived from the two measured oracle rates (GEMM 1447 GFLOP, attention 631 GFLOP), not run as a block"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
