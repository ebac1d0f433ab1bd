#!/usr/bin/env python3
"""Benchmark of the dense-kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-others]

A "step" is one launch of the hot-path kernel over one batch of seeded synthetic input that is
already resident in HBM.  The headline workload is the fp16 NT GEMM 8192^3 with fp16 output
(the configuration the TFLOP/s / %-of-MFMA-peak metric is quoted on); the other kernels of the
path (flash-attention prefill, paged decode, MXFP4 GEMM, remaining GEMM shapes) are measured in
the same run and reported under "others".  Prints exactly one JSON line.

Timing: W untimed warm-up steps and about 0.3 s more of untimed launches (until the GPU's clocks have settled:
"settle_ms" in the output), then exactly K steps, replayed as one HIP graph, bracketed by
torch.cuda.synchronize() on both sides (wall clock -> value / ms_per_step) and, inside the same
region, by a HIP event pair on the launch stream (-> the average device time per launch used for the
roofline figure).  HBM-bound workloads whose operands would fit the 256 MiB memory-side cache rotate over
enough copies of them that every timed launch streams from HBM.  The legs of the metric (GEMM, causal and
non-causal prefill, MXFP4 GEMM, decode) each carry a "cpu_baseline": the CPU restatement of the same
computation timed on a bounded sample on the host cores in the same run.

Calibration workloads (run only when named): library_gemm_8192 (torch.mm, the vendor library, on the headline shape), copy_1GiB (what the HBM counters read for a known copy) and
mfma_{f16,f16x16,fp4}_regloop_{zeros,benchmark} (what the MFMA unit sustains from registers on all-zero operands
and on operands drawn like the benchmark's: the measured ceiling beside the datasheet peak).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import platform
import sys
import time

import torch

PEAK_F16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_FP4_TFLOPS = 10100.0  # MI355X dense fp4 MFMA
PEAK_FP8_TFLOPS = 5000.0   # MI355X dense fp8 MFMA
PEAK_FP6_TFLOPS = 10100.0  # MI355X dense fp6 MFMA (the fp4 rate)
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

METRIC = "TFLOP/s & %MFMA peak (f16 GEMM, causal FA, MXFP4 GEMM); decode HBM GB/s"

# HBM bytes per launch measured with `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` (KiB per
# dispatch, scaled by what the same counters read for a copy kernel of known size); filled in from
# the summaries kept under profiles/.  None = not measured.
MEASURED_TRAFFIC_BYTES: dict[str, float | None] = {
    "gemm_8192": 1.754e9,              # 1545 MiB read + 128 MiB written: each of the 8 XCD L2s fetches its own copy of
                                       # the panels its 4x8 block of output tiles needs (12 panels x 4 MiB x 4 rounds x 8)
    "gemm_4096": 2.438e8,
    "gemm_2048x10240x8192": 6.973e8,   # of which 128 MiB are the strip's fp32 partial products, written and read once
    "gemm_2048x57344x8192": 3.062e9,
    "gemm_1024_f32out": 1.681e7,
    "gemm_bf16_8192": 1.754e9,
    "gemm_16x8192x8192": 1.366e8,
    "gemm_64x8192x8192": 1.439e8,
    "gemm_200x4096x4096": 4.980e7,
    "gemm_1000x1000x1024": 1.438e7,
    "gemm_1024x8192x8192": 3.644e8,
    "fa_causal": 3.537e8,
    "fa_noncausal": 2.686e8,
    "decode": 1.177e9,
    "fa_causal_bf16": 3.531e8,
    "decode_bf16": 1.177e9,
    "mxfp4_4096x8192x8192": 2.958e8,
    "mxfp4_32x8192x8192": 3.739e7,
    "mxfp4_quantize_16384x16384": 6.796e8,
    "mxfp8_quantize_16384x16384": 8.138e8,
    "mxfp6_quantize_16384x16384": 7.466e8,
    "paged_prefill": 6.832e8,
    "mxfp8_4096x8192x8192": 4.972e8,
    "mxfp6_4096x8192x8192": 3.819e8,
}


SETTLE_MS = 300.0  # untimed launches before the timed region, by device time


def settle_clocks(fn, budget_ms: float = SETTLE_MS) -> int:
    """Keeps calling `fn` (one launch, or one replay of the captured steps), untimed, until about `budget_ms` of device
    time have passed; returns the call count.  An idle GPU's power management takes tens of milliseconds of sustained
    work to reach the clocks it will hold, and a kernel of 0.1-0.3 ms measured right after a handful of warm-up launches
    reads 10-20 % off its sustained rate in either direction.  The W warm-up steps of the command line come first and
    are not replaced by this."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    done, batch = 0, 4
    torch.cuda.synchronize()
    e0.record()
    while True:
        for _ in range(batch):
            fn()
        done += batch
        e1.record()
        e1.synchronize()
        spent = e0.elapsed_time(e1)
        if spent >= budget_ms or done >= 20000:
            return done
        per_launch = max(spent / done, 1e-4)
        batch = max(4, min(2000, int((budget_ms - spent) / per_launch / 2) + 1))  # halve the remainder: no long overshoot


def time_steps(fn, steps: int, warmup: int):
    """Returns (wall ms per step, device ms per launch, how the steps were launched).

    The K timed steps are captured once into a HIP graph and replayed, so that launches shorter than the
    host's per-call cost (a 15 us kernel behind a 40 us Python dispatch) are timed back to back on the
    device; the replay is bracketed by synchronize() for the wall clock and by one HIP event pair on the
    launch stream for the device time.  If capture fails the same K steps run eagerly, one event pair each.
    The settling phase comes AFTER the capture, as untimed replays of the same graph that run right up to the timed
    one: capturing and instantiating a graph leaves the GPU idle for long enough that its clocks fall back, and a
    kernel that runs at a high clock (few stalls, power to spare) then reads up to 10 % low over a 5 ms timed region.
    """
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    graph = None
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(steps):
                fn()
        graph.replay()  # untimed: first replay uploads the graph
        torch.cuda.synchronize()
    except Exception as exc:  # capture unsupported for this op: time eager launches
        print(f"bench.py: graph capture failed ({type(exc).__name__}: {exc}); timing eager launches", file=sys.stderr)
        graph = None
        torch.cuda.synchronize()
    if graph is not None:
        settle_clocks(graph.replay)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        return wall_ms, e0.elapsed_time(e1) / steps, "hip_graph"
    settle_clocks(fn)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, sum(s.elapsed_time(e) for s, e in ev) / steps, "eager"


# ---- workloads --------------------------------------------------------------------------------

MEMORY_SIDE_CACHE_BYTES = 256 << 20  # sits behind L2; a buffer set smaller than this is served from it on replays


def rotating(call, operand_sets):
    """A step function that takes the next operand set on every call, round robin.  HBM-bound workloads whose
    operands fit the memory-side cache are given several copies of them (more than the cache holds in total), so
    that every launch of the timed region streams from HBM; the launches captured into the replayed graph each
    bind their own set."""
    state = [0]

    def fn():
        k = state[0] % len(operand_sets)
        state[0] += 1
        return call(*operand_sets[k])
    return fn


def copies_beyond_cache(nbytes: float) -> int:
    return max(2, int(math.ceil(1.5 * MEMORY_SIDE_CACHE_BYTES / nbytes)))


def wl_gemm(M, N, K, out_dtype="float16", in_dtype=torch.float16):
    from oracle import inputs

    tag = "bf16" if in_dtype == torch.bfloat16 else "f16"

    def build(dev):
        a, b = inputs.gemm_inputs(M, N, K, dtype=in_dtype)
        ad, bd = a.to(dev), b.to(dev)
        flops = 2.0 * M * N * K
        out_b = 4 if out_dtype == "float32" else 2
        nbytes = 2.0 * (M * K + N * K) + out_b * M * N
        hbm_bound = M <= 64  # decode-shaped: the weights are streamed once, far below the fp16 ridge point (312 flop/B)
        fn = lambda: torch.ops.mi355.gemm_nt(ad, bd, out_dtype, -1)
        rotate = 1
        if hbm_bound and nbytes < MEMORY_SIDE_CACHE_BYTES:
            rotate = copies_beyond_cache(nbytes)
            sets = [(ad, bd)] + [(ad.clone(), bd.clone()) for _ in range(rotate - 1)]
            fn = rotating(lambda x, w: torch.ops.mi355.gemm_nt(x, w, out_dtype, -1), sets)
        return {
            "fn": fn,
            "work": nbytes if hbm_bound else flops, "bytes": nbytes, "flops": flops, "bound": "hbm" if hbm_bound else "mfma",
            "peak": PEAK_HBM_GBS if hbm_bound else PEAK_F16_TFLOPS, "unit": "GB/s" if hbm_bound else "TFLOP/s",
            "dtype": tag, "cpu": lambda: cpu_gemm(a, b, M, N, K),
            "config": {"workload": f"gemm_{tag}_nt_{M}x{N}x{K}_{'f32' if out_dtype == 'float32' else tag}out",
                       "M": M, "N": N, "K": K, "layout": "NT", "accumulate": "f32", "out": out_dtype, "seed": 10,
                       "operand_sets_rotated": rotate},
        }
    return build


def wl_attention(causal, B=2, H=32, S=4096, D=128, bf16=False):
    from oracle import inputs

    def build(dev):
        q, k, v = inputs.attention_inputs(B, H, S, D)
        if bf16:
            q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
        qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
        flops = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0)
        return {
            "fn": lambda: torch.ops.mi355.flash_attn_fwd(qd, kd, vd, causal, 0.0),
            "work": flops, "bytes": 4 * 2.0 * B * H * S * D, "bound": "mfma", "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
            "dtype": "bf16" if bf16 else "f16", "cpu": lambda: cpu_attention(q, k, v, causal),
            "config": {"workload": f"flash_attn_fwd_{'bf16_' if bf16 else ''}{'causal' if causal else 'noncausal'}_B{B}_H{H}_S{S}_D{D}",
                       "B": B, "H": H, "S": S, "D": D, "causal": causal, "seed": 10},
        }
    return build


def wl_decode(bf16=False):
    from oracle import inputs

    def build(dev):
        q, kc, vc, bt, sl = inputs.paged_decode_inputs()
        if bf16:
            q, kc, vc = q.bfloat16(), kc.bfloat16(), vc.bfloat16()
        args = [t.to(dev) for t in (q, kc, vc, bt, sl)]
        total = int(sl.sum())
        kv_bytes = 4096.0 * total  # 2 (K,V) * 8 kv heads * 128 * 2 B per cached token, read once
        return {
            "fn": lambda: torch.ops.mi355.paged_decode_attn(*args, 0.0, 0),
            "work": kv_bytes, "bytes": kv_bytes, "bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "dtype": "bf16" if bf16 else "f16", "cpu": lambda: cpu_decode(q, kc, vc, bt, sl),
            "config": {"workload": f"paged_decode_{'bf16_' if bf16 else ''}64seq_32q8kv_D128_page16_ctx512-8192", "num_seqs": 64, "q_heads": 32,
                       "kv_heads": 8, "D": 128, "page": 16, "total_tokens": total, "seed": 10},
        }
    return build


def wl_paged_prefill(num_seqs=16, n_new=512, min_len=1024, max_len=8192):
    from oracle import inputs

    def build(dev):
        _, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=num_seqs, min_len=min_len, max_len=max_len)
        q = torch.randn((num_seqs, n_new, 32, 128), generator=torch.Generator().manual_seed(10)).half()
        args = [t.to(dev) for t in (q, kc, vc, bt, sl)]
        # query t of a sequence of length L sees L - n_new + t + 1 cached positions
        visible = sum(n_new * (int(L) - n_new) + n_new * (n_new + 1) // 2 for L in sl.tolist())
        flops = 4.0 * visible * 32 * 128
        return {
            "fn": lambda: torch.ops.mi355.paged_prefill_attn(*args, 0.0),
            "work": flops, "bytes": 4096.0 * int(sl.sum()) + 2 * q.numel() * 2.0, "bound": "mfma", "peak": PEAK_F16_TFLOPS,
            "unit": "TFLOP/s", "dtype": "f16", "cpu": lambda: cpu_paged_prefill(q, kc, vc, bt, sl),
            "config": {"workload": f"paged_prefill_{num_seqs}seq_{n_new}new_32q8kv_D128_page16_ctx{min_len}-{max_len}",
                       "num_seqs": num_seqs, "n_new": n_new, "q_heads": 32, "kv_heads": 8, "D": 128, "page": 16,
                       "total_tokens": int(sl.sum()), "seed": 10},
        }
    return build


def wl_mxfp4(M, N, K):
    from oracle import inputs

    def build(dev):
        a, asc, b, bsc = inputs.mxfp4_inputs(M, N, K)
        args = [t.to(dev) for t in (a, asc, b, bsc)]
        flops = 2.0 * M * N * K
        nbytes = (M + N) * K / 2 + (M + N) * K / 32 + 2.0 * M * N
        hbm_bound = flops / nbytes < 1250
        fn = lambda: torch.ops.mi355.mxfp4_gemm(*args, "bfloat16", -1)
        rotate = 1
        if hbm_bound and nbytes < MEMORY_SIDE_CACHE_BYTES:
            rotate = copies_beyond_cache(nbytes)
            sets = [tuple(args)] + [tuple(t.clone() for t in args) for _ in range(rotate - 1)]
            fn = rotating(lambda *ops: torch.ops.mi355.mxfp4_gemm(*ops, "bfloat16", -1), sets)
        return {
            "fn": fn,
            "work": nbytes if hbm_bound else flops, "bytes": nbytes, "flops": flops,
            "bound": "hbm" if hbm_bound else "mfma", "peak": PEAK_HBM_GBS if hbm_bound else PEAK_FP4_TFLOPS,
            "unit": "GB/s" if hbm_bound else "TFLOP/s", "dtype": "fp4(e2m1)+e8m0",
            "cpu": lambda: cpu_mxfp4(a, asc, b, bsc, M, N, K),
            "config": {"workload": f"mxfp4_gemm_{M}x{N}x{K}_bf16out", "M": M, "N": N, "K": K, "seed": 10,
                       "operand_sets_rotated": rotate},
        }
    return build


def wl_mxfp8(M, N, K):
    from oracle import inputs

    def build(dev):
        a, asc, b, bsc = inputs.mxfp8_inputs(M, N, K)
        args = [t.to(dev) for t in (a, asc, b, bsc)]
        flops = 2.0 * M * N * K
        nbytes = (M + N) * K * 1.0 + (M + N) * K / 32 + 2.0 * M * N
        return {
            "fn": lambda: torch.ops.mi355.mxfp8_gemm(*args, "bfloat16", -1),
            "work": flops, "bytes": nbytes, "flops": flops, "bound": "mfma", "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
            "dtype": "fp8(e4m3)+e8m0", "cpu": lambda: cpu_mxfp8(a, asc, b, bsc, M, N, K),
            "config": {"workload": f"mxfp8_gemm_{M}x{N}x{K}_bf16out", "M": M, "N": N, "K": K, "seed": 10},
        }
    return build


def wl_mxfp6(M, N, K):
    from oracle import inputs

    def build(dev):
        a, asc, b, bsc = inputs.mxfp6_inputs(M, N, K)
        args = [t.to(dev) for t in (a, asc, b, bsc)]
        flops = 2.0 * M * N * K
        nbytes = (M + N) * K * 0.75 + (M + N) * K / 32 + 2.0 * M * N
        return {
            "fn": lambda: torch.ops.mi355.mxfp6_gemm(*args, "e2m3", "bfloat16", -1),
            "work": flops, "bytes": nbytes, "flops": flops, "bound": "mfma", "peak": PEAK_FP6_TFLOPS, "unit": "TFLOP/s",
            "dtype": "fp6(e2m3)+e8m0", "cpu": lambda: cpu_mxfp6(a, asc, b, bsc, M, N, K),
            "config": {"workload": f"mxfp6_gemm_{M}x{N}x{K}_bf16out", "M": M, "N": N, "K": K, "seed": 10},
        }
    return build


def wl_quantize(rows, K):
    def build(dev):
        g = torch.Generator().manual_seed(10)
        x = (torch.randn(rows, K, generator=g) * 0.1).half()
        xd = x.to(dev)
        nbytes = rows * K * (2 + 0.5 + 1 / 32)
        return {
            "fn": lambda: torch.ops.mi355.mxfp4_quantize(xd),
            "work": nbytes, "bytes": nbytes, "bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "dtype": "f16 -> fp4(e2m1)+e8m0", "cpu": lambda: cpu_quantize(x),
            "config": {"workload": f"mxfp4_quantize_{rows}x{K}_f16in", "rows": rows, "K": K, "seed": 10},
        }
    return build


def wl_quantize8(rows, K):
    def build(dev):
        g = torch.Generator().manual_seed(10)
        x = (torch.randn(rows, K, generator=g) * 0.1).half()
        xd = x.to(dev)
        nbytes = rows * K * (2 + 1 + 1 / 32)
        return {
            "fn": lambda: torch.ops.mi355.mxfp8_quantize(xd),
            "work": nbytes, "bytes": nbytes, "bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "dtype": "f16 -> fp8(e4m3)+e8m0", "cpu": lambda: cpu_quantize8(x),
            "config": {"workload": f"mxfp8_quantize_{rows}x{K}_f16in", "rows": rows, "K": K, "seed": 10},
        }
    return build


def wl_quantize6(rows, K):
    def build(dev):
        g = torch.Generator().manual_seed(10)
        x = (torch.randn(rows, K, generator=g) * 0.1).half()
        xd = x.to(dev)
        nbytes = rows * K * (2 + 0.75 + 1 / 32)
        return {
            "fn": lambda: torch.ops.mi355.mxfp6_quantize(xd, "e2m3"),
            "work": nbytes, "bytes": nbytes, "bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "dtype": "f16 -> fp6(e2m3)+e8m0", "cpu": lambda: cpu_quantize6(x),
            "config": {"workload": f"mxfp6_quantize_{rows}x{K}_f16in", "rows": rows, "K": K, "seed": 10},
        }
    return build


def wl_copy(nbytes=1 << 30):
    """Plain device copy of a known size: the calibration point for the HBM traffic counters."""
    def build(dev):
        src = torch.full((nbytes // 2,), 1.0, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        return {
            "fn": lambda: dst.copy_(src),
            "work": 2.0 * nbytes, "bytes": 2.0 * nbytes, "bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "dtype": "f16", "cpu": lambda: cpu_copy(nbytes),
            "config": {"workload": f"copy_{nbytes >> 20}MiB", "bytes_read": nbytes, "bytes_written": nbytes},
        }
    return build


def wl_mfma_regloop(kind: str, data: str):
    """Register-only MFMA loop (mi355_calibrate_mfma): the rate the MFMA unit sustains on `data` with nothing else
    in the way.  "zeros" reads the issue-rate peak; "benchmark" uses operands drawn like the GEMM benchmarks'
    (fp16: N(0,1)*0.1; fp4: codes uniform over all 16 values, E8M0 exponents spread over [-8, 7])."""
    import ctypes

    from iree_turbine_amd import _lib

    def build(dev):
        g = torch.Generator().manual_seed(10)
        nbytes = 1 << 20
        if data == "zeros":
            ops = torch.zeros(nbytes, dtype=torch.uint8)
        elif kind.startswith("f16"):
            ops = (torch.randn(nbytes // 2, generator=g) * 0.1).half().view(torch.uint8)
        else:
            ops = torch.randint(0, 256, (nbytes,), generator=g, dtype=torch.uint8)
        opsd = ops.to(dev)
        workgroups, trips = (256, 1024) if kind.endswith("walk") else (512, 2000)  # one (512 registers per wave) or two workgroups of four waves per CU
        sink = torch.empty(workgroups * 256, dtype=torch.float32, device=dev)
        code = {"f16": 0, "f16x16": 3, "f16walk": 4, "f16x16walk": 5, "fp4walk": 6, "fp4x16walk": 7}.get(kind, 1 if data == "zeros" else 2)
        flop = ctypes.c_double(0.0)
        lib = _lib.load()

        def fn():
            rc = lib.mi355_calibrate_mfma(code, opsd.data_ptr(), nbytes, sink.data_ptr(), sink.numel(), workgroups, trips,
                                          ctypes.byref(flop), _lib.current_stream_ptr(dev))
            _lib.check(rc, "calibrate_mfma")
        fn()
        torch.cuda.synchronize()
        return {
            "fn": fn, "work": flop.value, "bytes": 0.0, "flops": flop.value, "bound": "mfma",
            "peak": PEAK_F16_TFLOPS if not kind.startswith("fp4") else PEAK_FP4_TFLOPS, "unit": "TFLOP/s",
            "dtype": "f16" if not kind.startswith("fp4") else "fp4(e2m1)+e8m0", "cpu": lambda: None,
            "config": {"workload": f"mfma_{kind}_regloop_{data}", "workgroups": workgroups, "trips": trips,
                       "instruction": {"f16": "v_mfma_f32_32x32x16_f16", "f16x16": "v_mfma_f32_16x16x32_f16",
                                       "f16walk": "v_mfma_f32_32x32x16_f16, 256 accumulators wandering around zero",
                                       "f16x16walk": "v_mfma_f32_16x16x32_f16, 256 accumulators wandering around zero",
                                       "fp4walk": "v_mfma_scale_f32_32x32x64_f8f6f4 (fp4 x fp4), 256 accumulators wandering around zero",
                                       "fp4x16walk": "v_mfma_scale_f32_16x16x128_f8f6f4 (fp4 x fp4), 256 accumulators wandering around zero"}.get(
                           kind, "v_mfma_scale_f32_32x32x64_f8f6f4 (fp4 x fp4)")},
        }
    return build


def wl_fa_issue_regloop(mode: str, waves_per_simd: int, data: str = "benchmark"):
    """The prefill tile's instruction mix out of registers (mi355_calibrate_fa_issue): what instruction issue alone
    lets the prefill kernel reach, at one or two waves per SIMD, on operands drawn like the attention benchmark's."""
    import ctypes

    from iree_turbine_amd import _lib

    def build(dev):
        g = torch.Generator().manual_seed(10)
        nbytes = 1 << 20
        if data == "zeros":  # the issue-rate reading: nothing toggles, the clock stays up
            opsd = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        else:
            opsd = (torch.randn(nbytes // 2, generator=g) * 0.35).half().view(torch.uint8).to(dev)  # scores of a few units
        workgroups, trips = 256 * waves_per_simd, 4000
        sink = torch.empty(workgroups * 256, dtype=torch.float32, device=dev)
        code = {"mix": 0, "nomax": 1, "mfma": 2, "vector": 3, "spread": 4, "stepwise": 5, "mix16": 6, "mfma16": 7}[mode]
        flop = ctypes.c_double(0.0)
        lib = _lib.load()

        def fn():
            rc = lib.mi355_calibrate_fa_issue(code, opsd.data_ptr(), nbytes, sink.data_ptr(), sink.numel(), workgroups, trips,
                                              ctypes.byref(flop), _lib.current_stream_ptr(dev))
            _lib.check(rc, "calibrate_fa_issue")
        fn()
        torch.cuda.synchronize()
        return {
            "fn": fn, "work": flop.value, "bytes": 0.0, "flops": flop.value, "bound": "mfma", "peak": PEAK_F16_TFLOPS,
            "unit": "TFLOP/s", "dtype": "f16", "cpu": lambda: None,
            "config": {"workload": f"fa_issue_regloop_{mode}_w{waves_per_simd}" + ("_zeros" if data == "zeros" else ""), "workgroups": workgroups, "trips": trips,
                       "waves_per_simd": waves_per_simd,
                       "per_wave_and_trip": {"mix": "32 MFMA 32x32x16, 32 v_exp_f32, 16 cvt_pk, 16 dot2, 16 v_max3 + test",
                                             "nomax": "32 MFMA 32x32x16, 32 v_exp_f32, 16 cvt_pk, 16 dot2",
                                             "mfma": "32 MFMA 32x32x16", "vector": "32 v_exp_f32, 16 cvt_pk, 16 dot2 (flop counted as if the MFMAs ran)",
                                             "spread": "the whole mix, vector work spread over all 32 MFMAs",
                                             "stepwise": "the whole mix, vector work behind the 16 score MFMAs, maximum chain behind the last 8 output MFMAs",
                                             "mix16": "64 MFMA 16x16x32 (the same flop), 32 v_exp_f32, 16 cvt_pk, 16 dot2",
                                             "mfma16": "64 MFMA 16x16x32 (the same flop)"}[mode]},
        }
    return build


WORKLOADS = {
    "gemm_8192": wl_gemm(8192, 8192, 8192),
    "gemm_4096": wl_gemm(4096, 4096, 4096),
    "gemm_2048x10240x8192": wl_gemm(2048, 10240, 8192),
    "gemm_2048x57344x8192": wl_gemm(2048, 57344, 8192),
    "gemm_1024_f32out": wl_gemm(1024, 1024, 1024, "float32"),
    "gemm_bf16_8192": wl_gemm(8192, 8192, 8192, "bfloat16", torch.bfloat16),
    "gemm_16x8192x8192": wl_gemm(16, 8192, 8192),
    "gemm_1024x8192x8192": wl_gemm(1024, 8192, 8192),  # 128 tiles: K split in two through the workspace entry point
    "gemm_512x8192x8192": wl_gemm(512, 8192, 8192),    # 64 tiles: four K ranges
    "gemm_64x8192x8192": wl_gemm(64, 8192, 8192),      # weight streaming with two row blocks
    "gemm_200x4096x4096": wl_gemm(200, 4096, 4096),    # a ragged number of rows: the last tile row cut inside the kernel
    "gemm_1000x1000x1024": wl_gemm(1000, 1000, 1024),  # ragged rows and columns: the last tile row and column cut inside the kernel
    "fa_causal": wl_attention(True),
    "fa_noncausal": wl_attention(False),
    "decode": wl_decode(),
    "fa_causal_bf16": wl_attention(True, bf16=True),
    "decode_bf16": wl_decode(bf16=True),
    "paged_prefill": wl_paged_prefill(),
    "mxfp4_4096x8192x8192": wl_mxfp4(4096, 8192, 8192),
    "mxfp4_32x8192x8192": wl_mxfp4(32, 8192, 8192),
    "mxfp4_quantize_16384x16384": wl_quantize(16384, 16384),
    "mxfp8_quantize_16384x16384": wl_quantize8(16384, 16384),
    "mxfp6_quantize_16384x16384": wl_quantize6(16384, 16384),
    "mxfp8_4096x8192x8192": wl_mxfp8(4096, 8192, 8192),
    "mxfp6_4096x8192x8192": wl_mxfp6(4096, 8192, 8192),
}
def wl_library_gemm(M, N, K):
    """The same NT product through torch.mm (hipBLASLt / rocBLAS): the vendor library's time beside this path's."""
    from oracle import inputs

    def build(dev):
        a, b = inputs.gemm_inputs(M, N, K)
        ad, bd = a.to(dev), b.to(dev)
        flops = 2.0 * M * N * K
        return {
            "fn": lambda: torch.mm(ad, bd.t()), "work": flops, "bytes": 2.0 * (M * K + N * K + M * N), "flops": flops,
            "bound": "mfma", "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s", "dtype": "f16", "cpu": lambda: None,
            "config": {"workload": f"library_torch_mm_f16_nt_{M}x{N}x{K}_f16out", "M": M, "N": N, "K": K, "seed": 10},
        }
    return build


CALIBRATION = {  # not part of the path: run only when named with --workload
    "library_gemm_8192": wl_library_gemm(8192, 8192, 8192),
    "library_gemm_2048x10240x8192": wl_library_gemm(2048, 10240, 8192),
    "library_gemm_1024x8192x8192": wl_library_gemm(1024, 8192, 8192),
    "library_gemm_512x8192x8192": wl_library_gemm(512, 8192, 8192),
    "library_gemm_1024": wl_library_gemm(1024, 1024, 1024),  # fp16 output: torch.mm has no fp32-output form
    "copy_1GiB": wl_copy(),
    "mfma_f16_regloop_zeros": wl_mfma_regloop("f16", "zeros"),
    "mfma_f16_regloop_benchmark": wl_mfma_regloop("f16", "benchmark"),
    "mfma_f16x16_regloop_zeros": wl_mfma_regloop("f16x16", "zeros"),
    "mfma_f16x16_regloop_benchmark": wl_mfma_regloop("f16x16", "benchmark"),
    "mfma_f16walk_regloop_zeros": wl_mfma_regloop("f16walk", "zeros"),
    "mfma_f16walk_regloop_benchmark": wl_mfma_regloop("f16walk", "benchmark"),
    "mfma_f16x16walk_regloop_zeros": wl_mfma_regloop("f16x16walk", "zeros"),
    "mfma_f16x16walk_regloop_benchmark": wl_mfma_regloop("f16x16walk", "benchmark"),
    "mfma_fp4walk_regloop_zeros": wl_mfma_regloop("fp4walk", "zeros"),
    "mfma_fp4walk_regloop_benchmark": wl_mfma_regloop("fp4walk", "benchmark"),
    "mfma_fp4x16walk_regloop_zeros": wl_mfma_regloop("fp4x16walk", "zeros"),
    "mfma_fp4x16walk_regloop_benchmark": wl_mfma_regloop("fp4x16walk", "benchmark"),
    **{f"fa_issue_regloop_{m}_w{w}": wl_fa_issue_regloop(m, w) for m in ("mix", "nomax", "mfma", "vector", "spread", "stepwise", "mix16", "mfma16") for w in (1, 2)},
    **{f"fa_issue_regloop_{m}_w{w}_zeros": wl_fa_issue_regloop(m, w, "zeros") for m in ("mix", "mfma", "vector", "spread", "stepwise", "mix16", "mfma16") for w in (1, 2)},
    "mfma_fp4_regloop_zeros": wl_mfma_regloop("fp4", "zeros"),
    "mfma_fp4_regloop_benchmark": wl_mfma_regloop("fp4", "benchmark"),
}
WORKLOADS_ALL = {**WORKLOADS, **CALIBRATION}
HEADLINE = "gemm_8192"


# ---- CPU baselines: the oracle, timed on the host cores on a bounded sample ------------------

def _time_cpu(fn, reps=3):
    fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return min(ts)


def cpu_copy(nbytes):
    src = torch.ones(nbytes // 8, dtype=torch.float16)
    dst = torch.empty_like(src)
    t = _time_cpu(lambda: dst.copy_(src))
    return {"value": 2.0 * (nbytes // 4) / t / 1e9, "unit": "GB/s", "sample": f"torch CPU copy of {nbytes >> 22} MiB"}


def cpu_quantize(x):
    from oracle import mxfp4 as om
    rows = 512
    t = _time_cpu(lambda: om.mxfp4_quantize_ref(x[:rows]), reps=2)
    return {"value": rows * x.shape[1] * (2 + 0.5 + 1 / 32) / t / 1e9, "unit": "GB/s",
            "sample": f"numpy quantiser on {rows} of the {x.shape[0]} rows, best of 2 after 1 warm-up"}


def cpu_quantize6(x):
    from oracle import mxfp6 as o6
    rows = 512
    t = _time_cpu(lambda: o6.mxfp6_quantize_ref(x[:rows], "e2m3"), reps=2)
    return {"value": rows * x.shape[1] * (2 + 0.75 + 1 / 32) / t / 1e9, "unit": "GB/s",
            "sample": f"numpy quantiser on {rows} of the {x.shape[0]} rows, best of 2 after 1 warm-up"}


def cpu_quantize8(x):
    from oracle import mxfp8 as o8
    rows = 512
    t = _time_cpu(lambda: o8.mxfp8_quantize_ref(x[:rows]), reps=2)
    return {"value": rows * x.shape[1] * (2 + 1 + 1 / 32) / t / 1e9, "unit": "GB/s",
            "sample": f"numpy quantiser on {rows} of the {x.shape[0]} rows, best of 2 after 1 warm-up"}


def cpu_gemm(a, b, M, N, K):
    from oracle import gemm as og
    rows = min(M, 1024)
    t = _time_cpu(lambda: og.gemm_nt_ref(a[:rows], b))
    return {"value": 2.0 * rows * N * K / t / 1e12, "unit": "TFLOP/s",
            "sample": f"torch fp32 matmul of A[0:{rows}] . B^T ({rows}x{N}x{K}), best of 3 after 1 warm-up"}


def cpu_attention(q, k, v, causal):
    from oracle import attention as oa
    qs, ks, vs = q[:1, :2], k[:1, :2], v[:1, :2]
    S, D = q.shape[2], q.shape[3]
    t = _time_cpu(lambda: oa.sdpa_torch(qs, ks, vs, is_causal=causal))
    flops = 4.0 * 2 * S * S * D * (0.5 if causal else 1.0)
    return {"value": flops / t / 1e12, "unit": "TFLOP/s",
            "sample": f"torch fp32 scaled_dot_product_attention on 2 of the {q.shape[0] * q.shape[1]} heads, best of 3 after 1 warm-up"}


def cpu_decode(q, kc, vc, bt, sl):
    """The oracle on the first 4 sequences, over a cache that holds only THEIR pages (renumbered): the oracle converts
    the cache it is handed to fp32 as a whole, and with the full 1.1 GB cache that conversion is what would be timed."""
    from oracle import paged_decode as op
    n = 4
    page = kc.shape[1]
    used = [int((int(sl[i]) + page - 1) // page) for i in range(n)]
    ids = torch.cat([bt[i, :used[i]].long() for i in range(n)])
    kc_s, vc_s = kc[ids].contiguous(), vc[ids].contiguous()
    bt_s = torch.zeros(n, max(used), dtype=bt.dtype)
    at = 0
    for i in range(n):
        bt_s[i, :used[i]] = torch.arange(at, at + used[i], dtype=bt.dtype)
        at += used[i]
    t = _time_cpu(lambda: op.paged_decode_ref(q[:n], kc_s, vc_s, bt_s, sl[:n]), reps=2)
    return {"value": 4096.0 * int(sl[:n].sum()) / t / 1e9, "unit": "GB/s",
            "sample": f"gather + dense fp32 attention for {n} of the {q.shape[0]} sequences over their own pages, best of 2 after 1 warm-up"}


def cpu_paged_prefill(q, kc, vc, bt, sl):
    from oracle import paged_decode as op
    n, t_new = 1, 64
    t = _time_cpu(lambda: op.paged_prefill_ref(q[:n, :t_new], kc, vc, bt[:n], sl[:n]), reps=2)
    L = int(sl[0])
    flops = 4.0 * (t_new * (L - t_new) + t_new * (t_new + 1) // 2) * q.shape[2] * q.shape[3]
    return {"value": flops / t / 1e12, "unit": "TFLOP/s",
            "sample": f"gather + dense fp32 causal attention for the last {t_new} tokens of 1 of the {q.shape[0]} sequences, best of 2 after 1 warm-up"}


def cpu_mxfp4(a, asc, b, bsc, M, N, K):
    from oracle import mxfp4 as om
    rows, cols = min(M, 256), min(N, 2048)
    t = _time_cpu(lambda: om.mxfp4_gemm_ref(a[:rows], asc[:rows], b[:cols], bsc[:cols]))
    flops = 2.0 * rows * cols * K
    return {"value": flops / t / 1e12, "unit": "TFLOP/s",
            "sample": f"table dequantise + torch fp32 matmul of a {rows}x{cols}x{K} corner, best of 3 after 1 warm-up"}


def cpu_mxfp6(a, asc, b, bsc, M, N, K):
    from oracle import mxfp6 as o6
    rows, cols = min(M, 256), min(N, 2048)
    t = _time_cpu(lambda: o6.mxfp6_gemm_ref(a[:rows], asc[:rows], b[:cols], bsc[:cols], "e2m3"))
    flops = 2.0 * rows * cols * K
    return {"value": flops / t / 1e12, "unit": "TFLOP/s",
            "sample": f"bit-unpack + table dequantise + torch fp32 matmul of a {rows}x{cols}x{K} corner, best of 3 after 1 warm-up"}


def cpu_mxfp8(a, asc, b, bsc, M, N, K):
    from oracle import mxfp8 as o8
    rows, cols = min(M, 256), min(N, 2048)
    t = _time_cpu(lambda: o8.mxfp8_gemm_ref(a[:rows], asc[:rows], b[:cols], bsc[:cols]))
    flops = 2.0 * rows * cols * K
    return {"value": flops / t / 1e12, "unit": "TFLOP/s",
            "sample": f"table dequantise + torch fp32 matmul of a {rows}x{cols}x{K} corner, best of 3 after 1 warm-up"}


# ---- driver -------------------------------------------------------------------------------------

def measure(name: str, dev, steps: int, warmup: int, with_cpu: bool):
    wl = WORKLOADS_ALL[name](dev)
    wall_ms, dev_ms, launch_mode = time_steps(wl["fn"], steps, warmup)
    scale = 1e9 if wl["unit"] == "GB/s" else 1e12
    achieved = wl["work"] / (dev_ms * 1e-3) / scale
    rec = {
        "workload": wl["config"]["workload"],
        "value": wl["work"] / (wall_ms * 1e-3) / scale,
        "unit": wl["unit"],
        "ms_per_step": wall_ms,
        "kernel_ms_avg": dev_ms,
        "launch": launch_mode,
        "dtype": wl["dtype"],
        "config": wl["config"],
        "roofline": {"bound": wl["bound"], "achieved": achieved, "peak": wl["peak"], "unit": wl["unit"],
                     "frac": achieved / wl["peak"], "traffic": MEASURED_TRAFFIC_BYTES.get(name)},
    }
    if "flops" in wl and wl["bound"] == "hbm":
        rec["tflops"] = wl["flops"] / (dev_ms * 1e-3) / 1e12
    if with_cpu:
        cpu = wl["cpu"]()
        if cpu is not None:
            cpu.update({"cores": torch.get_num_threads(), "kind": "port"})
            rec["cpu_baseline"] = cpu
    return rec


# Calibration runs that ride along with every default run, so that the line carries the vendor library's figure and the
# board's ceilings from the SAME box and session as the kernels' (boxes differ by a few per cent): hipBLASLt on the
# headline shape, the register-only MFMA loops on benchmark-like operands (plain and with a GEMM's register structure),
# the prefill tile's instruction mix out of registers.  They are not part of the path; `calibration: true` marks them.
CALIBRATION_IN_DEFAULT_RUN = ("library_gemm_8192", "library_gemm_1024", "mfma_f16_regloop_benchmark", "mfma_f16x16walk_regloop_benchmark",
                              "mfma_fp4_regloop_benchmark", "mfma_fp4x16walk_regloop_benchmark", "fa_issue_regloop_mix_w2",
                              "fa_issue_regloop_mfma_w2")

# the legs of the metric (GEMM, causal prefill, MXFP4 GEMM, decode): each gets its CPU baseline in the same run
CPU_TIMED = ("gemm_8192", "fa_causal", "fa_noncausal", "decode", "mxfp4_4096x8192x8192", "mxfp4_32x8192x8192")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed launches first; the clocks of an idle GPU take some tens of milliseconds of work to settle")
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS_ALL))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-others", action="store_true", help="measure only --workload")
    ap.add_argument("--library", default=None,
                    help="measure another build of the kernel library (python -m iree_turbine_amd.build -D... --out PATH); "
                         "a build with ablation switches computes wrong results and is named in the record")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); --gpus must be 1", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU fallback", file=sys.stderr)
        return 3

    if args.library:
        from pathlib import Path

        from iree_turbine_amd import _lib as _kernel_lib

        _kernel_lib.LIB_PATH = Path(args.library).resolve()
    import iree_turbine_amd  # noqa: F401  (registers torch.ops.mi355.*; raises if the library is missing)
    from iree_turbine_amd import _lib as _kernel_lib

    build_flags = _kernel_lib.build_flags()

    dev = torch.device("cuda:0")
    head = measure(args.workload, dev, args.steps, args.warmup, with_cpu=not args.no_cpu)
    others = []
    if not args.no_others:
        for name in WORKLOADS:
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            rec = measure(name, dev, args.steps, args.warmup, with_cpu=not args.no_cpu and name in CPU_TIMED)
            rec.pop("config")
            others.append(rec)
        for name in CALIBRATION_IN_DEFAULT_RUN:
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            rec = measure(name, dev, args.steps, args.warmup, with_cpu=False)
            rec.pop("config")
            rec["calibration"] = True
            others.append(rec)

    line = {
        "metric": METRIC,
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic (seeded torch CPU generator, seed 10; random-normal * 0.1 fp16 operands)",
        "config": head["config"],
        "kernel_ms_avg": head["kernel_ms_avg"],
        "launch": head["launch"],
        "settle_ms": SETTLE_MS,
        "roofline": head["roofline"],
        "cpu_baseline": head.get("cpu_baseline"),
        "host": {"cpu": platform.processor() or platform.machine(), "os_cpu_count": os.cpu_count(),
                 "torch_threads": torch.get_num_threads(), "gpu": torch.cuda.get_device_name(0)},
        "others": others,
    }
    # the vendor library's kernel on the same shape in the same run: boxes differ in the MFMA clock they sustain, so the
    # ratio says more about the kernel than the fraction of the datasheet peak does
    vendor = next((o for o in others if o.get("workload") == "library_torch_mm_f16_nt_8192x8192x8192_f16out"), None)
    if vendor and head["config"].get("workload") == "gemm_f16_nt_8192x8192x8192_f16out" and vendor.get("value"):
        line["vendor_same_run"] = {"workload": vendor["workload"], "value": vendor["value"], "unit": vendor["unit"],
                                   "ratio": head["value"] / vendor["value"]}
    if build_flags:  # not the product library: a timing-only build, its results are wrong on purpose
        line["library_ablations"] = build_flags
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
