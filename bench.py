#!/usr/bin/env python3
"""Benchmark of the gfx950 kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-extra]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The headline workload is the causal flash-attention forward the target is quoted on
(bf16, B=16 H=16 N=4096 D=128); the other configurations (attention backward, GQA decode, bf16 GEMM,
fp8 GEMM)
are measured in the same run and reported under "other_workloads" of the single JSON line.

FLOP / byte conventions (algorithmic work, fixed per configuration):
  attn_fwd_causal : 4*B*H*N^2*D / 2 FLOP (two GEMMs, causal half)           -> MFMA bf16 2.5 PFLOP/s
  attn_bwd_causal : 10*B*H*N^2*D / 2 FLOP (five GEMMs, causal half)         -> MFMA bf16 2.5 PFLOP/s
  gqa_decode      : bytes of K + V + Q + O                                   -> HBM 8 TB/s
  decode_step, rope_fwd, layernorm_residual, copy_kernel : bytes read + written      -> HBM 8 TB/s
  gemm_bf16       : 2*M*N*K FLOP                                             -> MFMA bf16 2.5 PFLOP/s
  gemm_fp8        : 2*M*N*K FLOP                                             -> MFMA fp8 5.0 PFLOP/s
Kernel durations are measured with HIP events on the stream the kernels are launched on.
The CPU baseline runs the reference's LibTorch call sequence (oracle/libtorch_path.py) on the host
cores of this box over a bounded sample of the same workload; it is a reported baseline only.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK = {"mfma_bf16": 2500.0, "mfma_fp8": 5000.0, "hbm": 8000.0}   # TFLOP/s, TFLOP/s, GB/s

# HBM bytes per launch of the dominant kernel, measured with `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` on this same script (one counter per run) and scaled by what the same counters
# read for the 1 GiB copy of --workload copy_1gib (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0); the raw
# figures are kept as text under profiles/.
TRAFFIC = {"attn_fwd_causal": 1_073_162_240 + 272_629_760, "gqa_decode": 1_090_820_096 + 270_336,
           "gemm_bf16": 202_589_594 + 33_554_432, "gemm_fp8": 810_477_568 + 136_314_880,
           # both backward kernels: dQ (1,713,229,824 + 276,824,064) + dK/dV (1,082,617,856 + 536,870,912)
           "attn_bwd_causal": 1_647_249_408 + 276_824_064 + 1_082_636_288 + 536_870_912,
           "rope_kernel<bf16>": 270_592_000 + 268_437_504,
           "layernorm_residual_kernel<2>": 268_521_472 + 268_435_456,
           "copy_kernel": 1_073_784_832 + 1_073_848_320,
           "decode_rope_append_kernel + gqa_decode_split_kernel<8>": 423_680 + 393_216 + 1_090_152_448 + 270_336}


def _events(torch, n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


# The device needs some tens of milliseconds of continuous work before its clocks settle (the first
# 50 attention launches after 10 warm-up launches run 2.5 % slower than the next 350; a 0.13 ms GEMM
# goes from 128 to 111 us per launch over its first 15 ms).  Every workload therefore runs untimed for
# this long before its W warm-up steps; the timed region is still exactly K steps.
PREWARM_MS = 80.0
# "randn" is the benchmark input.  "constant" fills every operand with 0.5: the same instruction stream
# with almost no bit toggling, which shows how much of the time is the device holding its clock down
# under the power the data draws (a diagnostic, never a headline number).
DATA = "randn"


def _normal(torch, *shape):
    if DATA == "constant":
        return torch.full(shape, 0.5, device="cuda")
    return torch.randn(*shape, device="cuda")


def time_steps(torch, fn, steps, warmup):
    """Runs the settle period, warmup + steps launches of fn on the current stream; returns (wall ms/step, event ms/step)."""
    t_end = time.perf_counter() + PREWARM_MS * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = _events(torch, 2)
    t0 = time.perf_counter()
    ev[0].record()
    for _ in range(steps):
        fn()
    ev[1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, ev[0].elapsed_time(ev[1]) / steps


# ------------------------------------------------------------------------------- workloads

def wl_attn(torch, tyr, steps, warmup, cpu):
    B, H, N, D = 16, 16, 4096, 128
    torch.manual_seed(0)
    q, k, v = (_normal(torch, B, H, N, D).to(torch.bfloat16) for _ in range(3))
    sc = 1.0 / math.sqrt(D)
    fn = lambda: tyr.flash_attn_fwd(q, k, v, causal=True, scale=sc)
    wall, ms = time_steps(torch, fn, steps, warmup)
    flop = 4.0 * B * H * N * N * D / 2.0
    tf = flop / (ms * 1e-3) / 1e12
    res = {
        "metric": "attn fwd TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "causal flash-attention forward, bf16, B=16 H=16 N=4096 D=128, O + LSE",
                   "flop_convention": "4*B*H*N^2*D/2 (causal half)", "scale": "1/sqrt(128)"},
        "roofline": {"bound": "mfma", "kernel": "flash_attn_fwd_kernel<128,true>", "achieved": tf,
                     "peak": PEAK["mfma_bf16"], "unit": "TFLOP/s", "frac": tf / PEAK["mfma_bf16"],
                     "traffic": TRAFFIC["attn_fwd_causal"]},
    }
    if cpu:
        from oracle import libtorch_path as lt
        hs = 16                                    # sample: one batch entry (16 of the 256 heads)
        qc, kc, vc = (t[:1, :hs].cpu() for t in (q, k, v))
        lt.sdpa_4d(qc[:, :2], kc[:, :2], vc[:, :2], True)   # warm-up
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10 and reps < 400):      # about 10 s of host work
            lt.sdpa_4d(qc, kc, vc, True)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": (4.0 * hs * N * N * D / 2.0) / dt / 1e12, "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU scaled_dot_product_attention(is_causal) on 1 of 16 batch "
                                         f"entries (16 heads, N=4096, D=128, bf16), {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_attn_bwd(torch, tyr, steps, warmup, cpu):
    B, H, N, D = 16, 16, 4096, 128
    torch.manual_seed(0)
    q, k, v, g = (_normal(torch, B, H, N, D).to(torch.bfloat16) for _ in range(4))
    sc = 1.0 / math.sqrt(D)
    o, lse = tyr.flash_attn_fwd(q, k, v, causal=True, scale=sc)
    fn = lambda: tyr.flash_attn_bwd(q, k, v, o, lse, g, causal=True, scale=sc)
    wall, ms = time_steps(torch, fn, steps, warmup)
    flop = 10.0 * B * H * N * N * D / 2.0
    tf = flop / (ms * 1e-3) / 1e12
    res = {
        "metric": "attn bwd TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "causal flash-attention backward, bf16, B=16 H=16 N=4096 D=128, dQ + dK + dV",
                   "flop_convention": "10*B*H*N^2*D/2 (five GEMMs, causal half); the two kernels execute seven",
                   "scale": "1/sqrt(128)"},
        "roofline": {"bound": "mfma", "kernel": "flash_attn_bwd_dq_kernel<128,true> + flash_attn_bwd_dkv_kernel<128,true>",
                     "achieved": tf, "peak": PEAK["mfma_bf16"], "unit": "TFLOP/s", "frac": tf / PEAK["mfma_bf16"],
                     "traffic": TRAFFIC.get("attn_bwd_causal")},
    }
    if cpu:
        from oracle import libtorch_path as lt
        hs = 4                                     # sample: 4 of the 256 heads
        qc, kc, vc, gc = (t[:1, :hs].cpu() for t in (q, k, v, g))
        lt.sdpa_4d_backward(qc[:, :1], kc[:, :1], vc[:, :1], gc[:, :1], True)   # warm-up
        reps, t0 = 0, time.perf_counter()
        while reps < 2 or (time.perf_counter() - t0 < 10 and reps < 20):
            lt.sdpa_4d_backward(qc, kc, vc, gc, True)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": (14.0 * hs * N * N * D / 2.0) / dt / 1e12, "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU autograd of scaled_dot_product_attention(is_causal), forward + "
                                         f"backward (14*N^2*D/2 FLOP per head), f32, 4 heads of N=4096 D=128, "
                                         f"{reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_decode(torch, tyr, steps, warmup, cpu):
    B, Hq, Hkv, L, D = 32, 32, 8, 8192, 128
    torch.manual_seed(1)
    q = torch.randn(B, Hq, 1, D, device="cuda").to(torch.bfloat16)
    # rotate over 4 independent caches (1.07 GB each) so no launch finds its K/V in the 256 MB last-level cache
    caches = [(torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16),
               torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)) for _ in range(4)]
    sc = 1.0 / math.sqrt(D)
    it = [0]

    def fn():
        k, v = caches[it[0] % len(caches)]
        it[0] += 1
        return tyr.gqa_decode(q, k, v, scale=sc)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 2 * B * Hkv * L * D * 2 + 2 * B * Hq * D * 2
    gbs = nbytes / (ms * 1e-3) / 1e9
    res = {
        "metric": "decode attn GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "GQA decode attention, bf16, batch 32, 32 q heads, 8 kv heads, D=128, KV length 8192",
                   "bytes_convention": "K + V + Q + O = 1,074,266,112 B (split partials excluded)",
                   "num_splits": int(__import__("tyr_amd._lib", fromlist=["load"]).load()
                                     .tyr_hip_gqa_decode_auto_splits(B, Hkv, L)),
                   "note": "one split per (batch, kv head) at this shape: the first pass writes O and LSE itself"},
        "roofline": {"bound": "hbm", "kernel": "gqa_decode_split_kernel<8>", "achieved": gbs,
                     "peak": PEAK["hbm"], "unit": "GB/s", "frac": gbs / PEAK["hbm"], "traffic": TRAFFIC["gqa_decode"]},
    }
    if cpu:
        from oracle import libtorch_path as lt
        nb = 4                                     # sample: 4 of the 32 sequences
        qc = q[:nb].cpu()
        kc, vc = (t[:nb].cpu() for t in caches[0])
        lt.sdpa_gqa_qkv(qc[:1], kc[:1], vc[:1])
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 8 and reps < 50):
            lt.sdpa_gqa_qkv(qc, kc, vc)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": nbytes * nb / B / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                               "kind": "port",
                               "sample": f"LibTorch CPU repeat_interleave + scaled_dot_product_attention on {nb} of 32 "
                                         f"sequences, {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_gemm_bf16(torch, tyr, steps, warmup, cpu):
    M = N = K = 4096
    torch.manual_seed(2)
    a = (_normal(torch, M, K) * K ** -0.25).to(torch.bfloat16)
    b = (_normal(torch, K, N) * K ** -0.25).to(torch.bfloat16)
    fn = lambda: tyr.gemm_bf16(a, b)
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    res = {
        "metric": "GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "bf16 GEMM M=N=K=4096, row-major A and B, f32 accumulate, bf16 out",
                   "input_std": "K^-1/4 = 0.125"},
        "roofline": {"bound": "mfma", "kernel": "gemm_bf16_fast_kernel<false>", "achieved": tf,
                     "peak": PEAK["mfma_bf16"], "unit": "TFLOP/s", "frac": tf / PEAK["mfma_bf16"],
                     "traffic": TRAFFIC["gemm_bf16"]},
    }
    if cpu:
        from oracle import libtorch_path as lt
        ac, bc = a.cpu(), b.cpu()
        lt.mm(ac[:256], bc)
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 8 and reps < 50):
            lt.mm(ac, bc)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": 2.0 * M * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "port", "sample": f"LibTorch CPU torch.mm (bf16) on the full 4096^3 problem, "
                                                         f"{reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_gemm_fp8(torch, tyr, steps, warmup, cpu):
    M = N = K = 8192
    torch.manual_seed(3)
    aq, sa = tyr.quantize_e4m3(_normal(torch, M, K))
    bq, sb = tyr.quantize_e4m3(_normal(torch, K, N))
    fn = lambda: tyr.gemm_fp8(aq, bq, sa, sb)
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    res = {
        "metric": "GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "fp8_e4m3",
        "config": {"workload": "fp8 e4m3 GEMM M=N=K=8192, per-tensor f32 scales, bf16 out"},
        "roofline": {"bound": "mfma", "kernel": "gemm_fp8_fast_kernel<false>", "achieved": tf,
                     "peak": PEAK["mfma_fp8"], "unit": "TFLOP/s", "frac": tf / PEAK["mfma_fp8"],
                     "traffic": TRAFFIC["gemm_fp8"]},
    }
    if cpu:
        from oracle import libtorch_path as lt
        rows = 1024                                # sample: 1/8 of the rows of A
        ac, bc = aq[:rows].cpu(), bq.cpu()
        lt.fp8_mm(ac[:64], bc, sa, sb)
        reps, t0 = 0, time.perf_counter()
        while reps < 2 or (time.perf_counter() - t0 < 8 and reps < 20):
            lt.fp8_mm(ac, bc, sa, sb)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": 2.0 * rows * N * K / dt / 1e12, "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU dequantise + f32 torch.mm on {rows} of 8192 rows of A, "
                                         f"{reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def _hbm_result(metric, workload, kernel, nbytes, ms, wall, dtype, extra=None):
    gbs = nbytes / (ms * 1e-3) / 1e9
    cfg = {"workload": workload, "bytes_convention": f"{nbytes:,} B read + written per launch"}
    if extra:
        cfg.update(extra)
    return {"metric": metric, "value": gbs, "unit": "GB/s", "ms_per_step": ms, "wall_ms_per_step": wall, "dtype": dtype,
            "config": cfg,
            "roofline": {"bound": "hbm", "kernel": kernel, "achieved": gbs, "peak": PEAK["hbm"], "unit": "GB/s",
                         "frac": gbs / PEAK["hbm"], "traffic": TRAFFIC.get(kernel)}}


def _cpu_time(fn, budget=6.0, max_reps=30):
    fn()
    reps, t0 = 0, time.perf_counter()
    while reps < 2 or (time.perf_counter() - t0 < budget and reps < max_reps):
        fn()
        reps += 1
    return (time.perf_counter() - t0) / reps, reps


def wl_rope(torch, tyr, steps, warmup, cpu):
    from oracle import libtorch_path as lt
    B, S, H, D = 16, 4096, 16, 128
    torch.manual_seed(0)
    xs = [torch.randn(B, S, H, D, device="cuda").to(torch.bfloat16) for _ in range(3)]   # 268 MB each, rotated
    cos, sin = (t.cuda() for t in lt.compute_rotary_freqs(S, D))
    it = [0]

    def fn():
        it[0] += 1
        return tyr.rope_fwd(xs[it[0] % 3], cos, sin)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 2 * B * S * H * D * 2 + 2 * S * (D // 2) * 4
    res = _hbm_result("rotary GB/s", "rotary embedding, bf16 [16,4096,16,128], cos/sin f32 [4096,64]",
                      "rope_kernel<bf16>", nbytes, ms, wall, "f32 arithmetic on bf16 data")
    if cpu:
        xc = xs[0][:1].cpu()
        dt, reps = _cpu_time(lambda: lt.apply_rotary_emb(xc, cos.cpu(), sin.cpu()))
        res["cpu_baseline"] = {"value": nbytes / B / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU slice/mul/sub/cat sequence on 1 of 16 batch entries, {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_layernorm(torch, tyr, steps, warmup, cpu):
    from oracle import libtorch_path as lt
    rows, d = 65536, 1024
    torch.manual_seed(0)
    xs = [(torch.rand(rows, d, device="cuda").to(torch.bfloat16), torch.rand(rows, d, device="cuda").to(torch.bfloat16))
          for _ in range(3)]
    w, b = torch.rand(d, device="cuda").to(torch.bfloat16), torch.rand(d, device="cuda").to(torch.bfloat16)
    it = [0]

    def fn():
        it[0] += 1
        x, r = xs[it[0] % 3]
        return tyr.layernorm_residual(x, r, w, b, 1e-5)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 4 * rows * d * 2 + 2 * d * 2
    res = _hbm_result("layernorm GB/s", "fused residual + LayerNorm, bf16, 65536 rows of 1024",
                      "layernorm_residual_kernel<2>", nbytes, ms, wall, "f32 arithmetic on bf16 data")
    if cpu:
        xc, rc = (t.cpu() for t in xs[0])            # all rows: a slice that fits the host caches would flatter the CPU
        wc, bc = w.cpu(), b.cpu()
        dt, reps = _cpu_time(lambda: lt.layer_norm_residual(xc, rc, wc, bc, 1e-5))
        res["cpu_baseline"] = {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU add + layer_norm on all 65536 rows, {reps} reps, {dt * 1e3:.1f} ms each"}
    return res


def wl_copy_kernel(torch, tyr, steps, warmup, cpu):
    n = 1 << 30
    srcs = [torch.empty(n, dtype=torch.uint8, device="cuda").random_() for _ in range(2)]
    it = [0]

    def fn():
        it[0] += 1
        return tyr.copy(srcs[it[0] % 2])
    wall, ms = time_steps(torch, fn, steps, warmup)
    res = _hbm_result("copy GB/s", "device copy kernel, 1 GiB", "copy_kernel", 2 * n, ms, wall, "u8")
    if cpu:
        sc = srcs[0][: n // 8].cpu()
        dt, reps = _cpu_time(lambda: sc.clone())
        res["cpu_baseline"] = {"value": 2 * (n // 8) / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU clone of 128 MiB, {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_decode_step(torch, tyr, steps, warmup, cpu):
    """The decode step's cache update followed by attention over the cache (forwardStep order)."""
    from oracle import libtorch_path as lt
    B, Hq, Hkv, L, D = 32, 32, 8, 8192, 128
    torch.manual_seed(1)
    q = torch.randn(B, Hq, 1, D, device="cuda").to(torch.bfloat16)
    kn, vn = (torch.randn(B, Hkv, 1, D, device="cuda").to(torch.bfloat16) for _ in range(2))
    caches = [(torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16),
               torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)) for _ in range(4)]
    cos_t, sin_t = lt.compute_rotary_freqs(L, D)
    cos, sin = cos_t[L - 1:].contiguous().cuda(), sin_t[L - 1:].contiguous().cuda()
    sc = 1.0 / math.sqrt(D)
    it = [0]

    def fn():
        k, v = caches[it[0] % len(caches)]
        it[0] += 1
        qr = tyr.decode_rope_append(q, kn, vn, cos, sin, k, v, L - 1)
        return tyr.gqa_decode(qr, k, v, scale=sc, kv_len=L)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 2 * B * Hkv * L * D * 2 + 2 * B * Hq * D * 2
    res = _hbm_result("decode step GB/s", "decode step: rotate q/k + append k/v to the cache (position 8191) + GQA decode "
                      "attention over 8192 cached rows, bf16, batch 32, 32 q heads, 8 kv heads, D=128",
                      "decode_rope_append_kernel + gqa_decode_split_kernel<8>", nbytes, ms, wall, "bf16",
                      {"bytes_convention": "bytes of the attention pass (K + V + Q + O); the append moves 0.4 MB more"})
    return res


def wl_copy(torch, tyr, steps, warmup, cpu):
    """Counter calibration only: a plain device copy of exactly 1 GiB (reads 2^30 B, writes 2^30 B)."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    wall, ms = time_steps(torch, lambda: dst.copy_(src), steps, warmup)
    gbs = 2.0 * n / (ms * 1e-3) / 1e9
    return {"metric": "copy GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "wall_ms_per_step": wall,
            "dtype": "u8", "config": {"workload": "device-to-device copy of 1 GiB (counter calibration)"},
            "roofline": {"bound": "hbm", "kernel": "torch elementwise copy", "achieved": gbs, "peak": PEAK["hbm"],
                         "unit": "GB/s", "frac": gbs / PEAK["hbm"], "traffic": 2.0 * n}}


def wl_dsl_simple_gemm(torch, tyr, steps, warmup, cpu):
    """The reference's example GEMM program (Tyr/GPU/Kernels/Examples.lean:23-65) emitted for gfx950 by
    tyr_amd.dsl: one 64x64 tile per one-wave workgroup, single-buffered, as the program is written."""
    from tyr_amd.dsl import kernels, runtime
    M = N = 8192
    K = 512
    torch.manual_seed(0)
    a = (_normal(torch, M, K) * K ** -0.25).to(torch.bfloat16)
    b = (_normal(torch, K, N) * K ** -0.25).to(torch.bfloat16)
    c = torch.zeros(M, N, device="cuda")
    kern = kernels.simpleGemm()
    fn = lambda: runtime.launch(kern, [a, b, c, M, N, K], grid=(N // 64, M // 64, 1), block=(32, 1, 1))   # one warp of the reference = one wave
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    return {"metric": "emitted GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
            "dtype": "bf16",
            "config": {"workload": "tile-DSL program simpleGemm emitted for gfx950, bf16 x bf16 -> f32, M=N=8192 K=512, "
                                   "64x64 tile per one-wave workgroup"},
            "roofline": {"bound": "mfma", "kernel": "simpleGemm (emitted)", "achieved": tf, "peak": PEAK["mfma_bf16"],
                         "unit": "TFLOP/s", "frac": tf / PEAK["mfma_bf16"], "traffic": None}}


WORKLOADS = {"attn_fwd_causal": wl_attn, "attn_bwd_causal": wl_attn_bwd, "gqa_decode": wl_decode, "gemm_bf16": wl_gemm_bf16,
             "gemm_fp8": wl_gemm_fp8, "decode_step": wl_decode_step, "rope_fwd": wl_rope, "layernorm_residual": wl_layernorm,
             "copy_kernel": wl_copy_kernel, "dsl_simple_gemm": wl_dsl_simple_gemm}
CALIBRATION = {"copy_1gib": wl_copy}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="attn_fwd_causal", choices=sorted(WORKLOADS) + sorted(CALIBRATION))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-extra", action="store_true", help="measure only --workload")
    ap.add_argument("--settle-ms", type=float, default=PREWARM_MS,
                    help="untimed work before the warm-up steps of every workload, in milliseconds")
    ap.add_argument("--data", default="randn", choices=["randn", "constant"],
                    help="operand values of the attention and GEMM workloads; 'constant' is a power diagnostic")
    args = ap.parse_args()
    globals()["PREWARM_MS"] = args.settle_ms
    globals()["DATA"] = args.data
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        return 2

    import torch
    import tyr_amd
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False).", file=sys.stderr)
        return 3
    torch.cuda.set_device(0)
    info = tyr_amd.device_info(0)

    if args.workload in CALIBRATION:
        args.no_extra = True
    head = {**WORKLOADS, **CALIBRATION}[args.workload](torch, tyr_amd, args.steps, args.warmup, not args.no_cpu)
    line = {
        "metric": head["metric"], "value": round(head["value"], 3), "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "settle_ms_before_warmup": PREWARM_MS,
        "ms_per_step": round(head["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic" if DATA == "randn" else "synthetic, every operand 0.5 (power diagnostic, not the benchmark input)",
        "config": head["config"], "roofline": head["roofline"],
        "cpu_baseline": head.get("cpu_baseline"), "wall_ms_per_step": round(head["wall_ms_per_step"], 5),
        "device": info,
    }
    if not args.no_extra:
        others = []
        for name, fn in WORKLOADS.items():
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            try:
                r = fn(torch, tyr_amd, max(10, args.steps // 2), max(3, args.warmup // 2), not args.no_cpu)
            except Exception as e:                      # a side workload must not take the headline line with it
                r = {"error": f"{type(e).__name__}: {e}"}
            r["workload"] = name
            others.append(r)
        line["other_workloads"] = others
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
