#!/usr/bin/env python3
"""Benchmark of the gfx950 kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-parity] [--no-extra]
                    [--details FILE]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The headline workload is the causal flash-attention forward the target is quoted on
(bf16, B=16 H=16 N=4096 D=128); the other configurations (attention backward, GQA decode, bf16 GEMM,
fp8 GEMM)
are measured in the same run.  Standard output carries ONE compact JSON line (a few KB): the headline
fields, a summary of every configuration of the benchmark under "baseline_configs" and of the remaining
workloads under "other_workloads" (time, rate, roofline fraction, HBM traffic, parity verdict, CPU figure
with core counts).  The full records (conventions, samples, notes) go to standard error as one JSON line
starting with {"details": and, with --details FILE, to that file.

FLOP / byte conventions (algorithmic work, fixed per configuration):
  attn_fwd_causal : 4*B*H*N^2*D / 2 FLOP (two GEMMs, causal half)           -> MFMA bf16 2.5 PFLOP/s
  attn_bwd_causal : 10*B*H*N^2*D / 2 FLOP (five GEMMs, causal half)         -> MFMA bf16 2.5 PFLOP/s
  gqa_decode      : bytes of K + V + Q + O                                   -> HBM 8 TB/s
  decode_step, rope_fwd, layernorm_residual, copy_kernel : bytes read + written      -> HBM 8 TB/s
  gemm_bf16       : 2*M*N*K FLOP                                             -> MFMA bf16 2.5 PFLOP/s
  gemm_fp8        : 2*M*N*K FLOP                                             -> MFMA fp8 5.0 PFLOP/s
Kernel durations are measured with HIP events on the stream the kernels are launched on.
Inputs follow the reference's recipe (Examples/GPU/RunFlashAttn.lean:19-58): torch.manual_seed on the
host, randn on the host in a fixed order, cast, copy to the device.  After its timed region every
workload checks a sample of the outputs it just produced against the CPU checker and reports the error
next to the figure ("parity": max-abs / relative Frobenius error, tolerance, sample), as the reference's
runners print their error beside the verdict (Examples/GPU/RunFlashAttn.lean:88-93).  The matrix-core
workloads also carry `roofline.sustained_peak`: the rate an MFMA-only loop reaches on this device with
normally distributed operands, measured in the same run (tyr_hip_mfma_sustain).
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
BWD_KERNELS = "flash_attn_bwd_dq_kernel<128,true> + flash_attn_bwd_dkv_kernel<128,true>"
TRAFFIC = {"attn_fwd_causal": 1_079_701_504 + 289_406_976, "gqa_decode": 1_090_820_096 + 270_336,
           "gemm_bf16": 202_589_594 + 33_554_432, "gemm_fp8": 810_477_568 + 136_314_880,
           # both backward kernels: dQ (1,713,229,824 + 276,824,064) + dK/dV (1,082,617,856 + 536,870,912)
           "attn_bwd_causal": 1_647_249_408 + 276_824_064 + 1_082_636_288 + 536_870_912,
           "rope_kernel<bf16>": 270_592_000 + 268_437_504,
           "layernorm_residual_kernel<2>": 268_521_472 + 268_435_456,
           "copy_kernel": 1_073_784_832 + 1_073_848_320,
           "decode_rope_append_kernel + gqa_decode_split_kernel<8>": 423_680 + 393_216 + 1_090_152_448 + 270_336,
           "gqa_decode_split4": 1_085_655_040 + 2_228_224 + 2_403_328 + 294_912,       # split pass + combine pass
           "gqa_decode_small_batch": 542_947_328 + 589_824 + 601_088 + 36_864,
           "dsl_simple_gemm": 77_063_987 + 268_435_456, "dsl_h100_gemm": 39_013_376 + 134_217_728,
           "dsl_lcf_attn": 655_022_080 + 50_331_648}


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
    """One f32 tensor of the benchmark input on the device.  "randn": drawn on the host from the generator the
    caller seeded with torch.manual_seed (the reference's recipe), then copied."""
    if DATA == "constant":
        return torch.full(shape, 0.5, device="cuda")
    return torch.randn(*shape).cuda()


def _bits(t):
    return t.detach().cpu().contiguous().view(__import__("torch").uint16).numpy().copy()


_SUSTAINED = {}


def sustained_peak(torch, kind):
    """TFLOP/s of an MFMA-only loop (no LDS, no memory, no vector work) on normally distributed operands:
    what the matrix cores of this device sustain with such data.  kind: "mfma_bf16" | "mfma_fp8"."""
    if kind in _SUSTAINED:
        return _SUSTAINED[kind]
    import ctypes
    from tyr_amd import _lib
    L = _lib.load()
    g = torch.Generator().manual_seed(1234)
    x = torch.randn(1 << 20, generator=g)
    ops = (x.to(torch.bfloat16) if kind == "mfma_bf16" else x.to(torch.float8_e4m3fn)).cuda()
    dtype = 0 if kind == "mfma_bf16" else 1
    wgs, iters = 256, 2000
    sink = torch.empty(wgs * 256, device="cuda")
    flop = ctypes.c_double()
    st = torch.cuda.current_stream().cuda_stream

    def fn():
        rc = L.tyr_hip_mfma_sustain(ops.data_ptr(), ops.numel() * ops.element_size(), dtype, wgs, iters,
                                    sink.data_ptr(), sink.numel() * sink.element_size(), ctypes.byref(flop), st)
        assert rc == 0, rc
    _, ms = time_steps(torch, fn, 20, 5)
    _SUSTAINED[kind] = {"value": flop.value / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
                        "how": f"tyr_hip_mfma_sustain: {wgs} workgroups x 4 waves, {iters} rounds of 16 "
                               f"{'32x32x16 bf16' if dtype == 0 else '32x32x64 e4m3'} MFMAs on randn operands, "
                               f"{ms:.3f} ms per launch, same run"}
    return _SUSTAINED[kind]


def _mfma_roofline(torch, kind, kernel, tf, traffic):
    sp = sustained_peak(torch, kind)
    return {"bound": "mfma", "kernel": kernel, "achieved": tf, "peak": PEAK[kind], "unit": "TFLOP/s",
            "frac": tf / PEAK[kind], "traffic": traffic,
            "sustained_peak": round(sp["value"], 1), "frac_of_sustained": tf / sp["value"], "sustained_how": sp["how"]}


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
# Every workload: fn(torch, tyr, steps, warmup, cpu, parity) -> dict.  `cpu` adds the LibTorch-CPU baseline,
# `parity` the check of a sample of the GPU outputs against the CPU checker (both outside the timed region;
# they are the only places that import `oracle`).

def _parity(max_abs=None, rel_fro=None, tol=None, sample="", **more):
    d = {k: (float(v) if v is not None else None) for k, v in (("max_abs", max_abs), ("rel_fro", rel_fro)) if v is not None}
    d.update({k: float(v) for k, v in more.items()})
    d["tol"] = tol
    d["sample"] = sample
    worst = max(float(v) for k, v in d.items() if k not in ("tol", "sample") and not k.startswith("tol_"))
    d["ok"] = bool(worst <= tol) if "ok" not in more else bool(more["ok"])
    return d


def wl_attn(torch, tyr, steps, warmup, cpu, parity):
    B, H, N, D = 16, 16, 4096, 128
    torch.manual_seed(0)
    q, k, v = (_normal(torch, B, H, N, D).to(torch.bfloat16) for _ in range(3))     # drawn in the order Q, K, V
    sc = 1.0 / math.sqrt(D)
    out = [None]

    def fn():
        out[0] = tyr.flash_attn_fwd(q, k, v, causal=True, scale=sc)
    wall, ms = time_steps(torch, fn, steps, warmup)
    flop = 4.0 * B * H * N * N * D / 2.0
    tf = flop / (ms * 1e-3) / 1e12
    # The two launch shapes of the forward, timed alternately after the headline's timed region (same box, same run).  A
    # comparison leg: it runs with the output check only, so that a profile taken with --no-parity holds the launches of the
    # default shape and nothing else.
    from tyr_amd import _lib
    L = _lib.load()
    default_shape = L.tyr_hip_flash_attn_fwd_persistent(0)
    L.tyr_hip_flash_attn_fwd_persistent(default_shape)
    pair = {"per_job": [], "persistent": []}
    if parity:
        for _ in range(3):
            for name, on in (("per_job", 0), ("persistent", 1)):
                L.tyr_hip_flash_attn_fwd_persistent(on)
                pair[name].append(time_steps(torch, fn, steps, 2)[1])
        L.tyr_hip_flash_attn_fwd_persistent(default_shape)
        fn()                                        # `out` holds a launch of the default shape again
    res = {
        "metric": "attn fwd TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "causal flash-attention forward, bf16, B=16 H=16 N=4096 D=128, O + LSE",
                   "flop_convention": "4*B*H*N^2*D/2 (causal half)", "scale": "1/sqrt(128)",
                   "inputs": "torch.manual_seed(0); Q, K, V = randn on the host in that order -> bf16 -> device",
                   "launch_shape": "persistent" if default_shape else "per_job",
                   "launch_shapes_ms": {k_: round(sorted(v_)[1], 5) for k_, v_ in pair.items()} if parity else None},
        "roofline": _mfma_roofline(torch, "mfma_bf16", "flash_attn_fwd_kernel<128,true>", tf, TRAFFIC["attn_fwd_causal"]),
    }
    if parity:
        import numpy as np
        import oracle
        o, lse = out[0]
        e_o = e_l = 0.0
        heads = ((0, 0), (15, 15))
        for (b, h) in heads:
            o64, l64 = oracle.attn_fwd_f64(_bits(q[b:b + 1, h:h + 1]), _bits(k[b:b + 1, h:h + 1]),
                                           _bits(v[b:b + 1, h:h + 1]), True, sc)
            e_o = max(e_o, float(np.abs(o[b, h].cpu().float().numpy() - o64[0, 0]).max()))
            e_l = max(e_l, float(np.abs(lse[b, h].cpu().numpy() - l64[0, 0]).max()))
        res["parity"] = _parity(tol=2e-2, max_abs_o=e_o, max_abs_lse=e_l,
                                sample=f"outputs of the last timed launch, heads {list(heads)}, all 4096 rows, against the "
                                       "float64 checker (oracle.attn_fwd_f64) on the same bf16 inputs")
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


def wl_attn_bwd(torch, tyr, steps, warmup, cpu, parity):
    B, H, N, D = 16, 16, 4096, 128
    torch.manual_seed(0)
    q, k, v, g = (_normal(torch, B, H, N, D).to(torch.bfloat16) for _ in range(4))
    sc = 1.0 / math.sqrt(D)
    o, lse = tyr.flash_attn_fwd(q, k, v, causal=True, scale=sc)
    out = [None]

    def fn():
        out[0] = tyr.flash_attn_bwd(q, k, v, o, lse, g, causal=True, scale=sc)
    wall, ms = time_steps(torch, fn, steps, warmup)
    flop = 10.0 * B * H * N * N * D / 2.0
    tf = flop / (ms * 1e-3) / 1e12
    res = {
        "metric": "attn bwd TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "causal flash-attention backward, bf16, B=16 H=16 N=4096 D=128, dQ + dK + dV",
                   "flop_convention": "10*B*H*N^2*D/2 (five GEMMs, causal half)",
                   "scale": "1/sqrt(128)"},
        "roofline": _mfma_roofline(torch, "mfma_bf16", BWD_KERNELS, tf, TRAFFIC.get("attn_bwd_causal")),
    }
    if parity:
        import numpy as np
        import oracle
        b, h = 3, 5
        sl = lambda t: _bits(t[b:b + 1, h:h + 1])
        want = oracle.attn_bwd_f64(sl(q), sl(k), sl(v), sl(g), True, sc)
        errs, rels = [], []
        for got, w_ in zip(out[0], want):
            gnp = got[b, h].cpu().float().numpy()
            errs.append(float(np.abs(gnp - w_[0, 0]).max()))
            rels.append(float(np.linalg.norm(gnp - w_[0, 0]) / np.linalg.norm(w_[0, 0])))
        res["parity"] = _parity(tol=3e-2, max_abs=max(errs), rel_fro=max(rels), tol_rel_fro=1e-2,
                                ok=max(errs) <= 3e-2 and max(rels) <= 1e-2,
                                sample=f"dQ, dK, dV of the last timed launch, head ({b},{h}), all rows, against the float64 "
                                       "checker (oracle.attn_bwd_f64); bars: the reference runner's allclose(3e-2) and "
                                       "relative Frobenius 1e-2")
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


def _decode_caches(torch, B, Hkv, L, D, n):
    """Cache 0 follows the seeded host recipe (it is the one the parity leg checks); the other n-1 exist only so
    that no launch finds its K/V in the 256 MB last-level cache, and are drawn on the device."""
    k0, v0 = (torch.randn(B, Hkv, L, D).to(torch.bfloat16).cuda() for _ in range(2))
    return [(k0, v0)] + [(torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16),
                          torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)) for _ in range(n - 1)]


def _wl_decode(torch, tyr, steps, warmup, cpu, parity, splits, shape=(32, 32, 8, 8192, 128)):
    B, Hq, Hkv, L, D = shape
    torch.manual_seed(1)
    q = torch.randn(B, Hq, 1, D).to(torch.bfloat16).cuda()
    caches = _decode_caches(torch, B, Hkv, L, D, 4 if B * Hkv * L * D * 4 > (64 << 20) else 8)
    sc = 1.0 / math.sqrt(D)
    it = [0]
    out = [None]

    def fn():
        k, v = caches[it[0] % len(caches)]
        it[0] += 1
        out[0] = tyr.gqa_decode(q, k, v, scale=sc, num_splits=splits)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 2 * B * Hkv * L * D * 2 + 2 * B * Hq * D * 2
    gbs = nbytes / (ms * 1e-3) / 1e9
    used = splits or int(__import__("tyr_amd._lib", fromlist=["load"]).load().tyr_hip_gqa_decode_auto_splits(B, Hkv, L))
    res = {
        "metric": "decode attn GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": f"GQA decode attention, bf16, batch {B}, {Hq} q heads, {Hkv} kv heads, D={D}, KV length {L}",
                   "bytes_convention": f"K + V + Q + O = {nbytes:,} B (split partials excluded)",
                   "num_splits": used,
                   "note": ("one split per (batch, kv head): the first pass writes O and LSE itself" if used == 1 else
                            f"{used} KV splits per (batch, kv head): split pass writes f32 partials (O, m, l), the "
                            "combine pass merges them with the LSE algebra; both passes are inside the timed step")},
        "roofline": {"bound": "hbm", "kernel": "gqa_decode_split_kernel<8>" + ("" if used == 1 else " + gqa_decode_combine_kernel"),
                     "achieved": gbs, "peak": PEAK["hbm"], "unit": "GB/s", "frac": gbs / PEAK["hbm"],
                     "traffic": {((32, 32, 8, 8192, 128), 1): TRAFFIC["gqa_decode"],
                                 ((32, 32, 8, 8192, 128), 4): TRAFFIC["gqa_decode_split4"],
                                 ((4, 32, 8, 32768, 128), 8): TRAFFIC["gqa_decode_small_batch"]}.get((shape, used))},
    }
    if parity:
        import numpy as np
        import oracle
        # the last launch read caches[(it-1) % n]; rerun on cache 0 (the seeded one) so the sample is reproducible
        o, lse = tyr.gqa_decode(q, caches[0][0], caches[0][1], scale=sc, num_splits=splits)
        e_o = e_l = 0.0
        seqs = sorted({0, B - 1})
        for b in seqs:
            wo, wl = oracle.gqa_decode(_bits(q[b:b + 1]), _bits(caches[0][0][b:b + 1]), _bits(caches[0][1][b:b + 1]), sc, used)
            wo32 = torch.from_numpy(wo.copy()).view(torch.bfloat16).float().numpy()
            e_o = max(e_o, float(np.abs(o[b:b + 1].cpu().float().numpy() - wo32).max()))
            e_l = max(e_l, float(np.abs(lse[b:b + 1].cpu().numpy() - wl).max()))
        res["parity"] = _parity(tol=2e-2, max_abs_o=e_o, max_abs_lse=e_l,
                                sample=f"sequences {seqs} (all {Hq} heads) of the seeded cache against the scalar C "
                                       f"restatement (oracle.gqa_decode, {used} splits)")
    if cpu:
        from oracle import libtorch_path as lt
        nb = min(4, B)                             # sample: 4 of the sequences
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
                               "sample": f"LibTorch CPU repeat_interleave + scaled_dot_product_attention on {nb} of {B} "
                                         f"sequences, {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_decode(torch, tyr, steps, warmup, cpu, parity):
    return _wl_decode(torch, tyr, steps, warmup, cpu, parity, 0)


def wl_decode_split4(torch, tyr, steps, warmup, cpu, parity):
    """The same configuration with the split-KV + LSE-combine path forced (4 splits, two kernels per step)."""
    return _wl_decode(torch, tyr, steps, warmup, False, parity, 4)


def wl_decode_small_batch(torch, tyr, steps, warmup, cpu, parity):
    """A shape where the library itself chooses several splits: batch 4, 32 q heads, 8 kv heads, 32768 cached rows."""
    return _wl_decode(torch, tyr, steps, warmup, False, parity, 0, shape=(4, 32, 8, 32768, 128))


def wl_gemm_bf16(torch, tyr, steps, warmup, cpu, parity):
    M = N = K = 4096
    torch.manual_seed(2)
    a = (_normal(torch, M, K) * K ** -0.25).to(torch.bfloat16)
    b = (_normal(torch, K, N) * K ** -0.25).to(torch.bfloat16)
    out = [None]

    def fn():
        out[0] = tyr.gemm_bf16(a, b)
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    res = {
        "metric": "GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16",
        "config": {"workload": "bf16 GEMM M=N=K=4096, row-major A and B, f32 accumulate, bf16 out",
                   "input_std": "K^-1/4 = 0.125"},
        "roofline": _mfma_roofline(torch, "mfma_bf16", "gemm_bf16_fast_kernel<false>", tf, TRAFFIC["gemm_bf16"]),
    }
    if parity:
        import numpy as np
        import oracle
        rows = list(range(0, 32)) + list(range(M - 32, M))
        idx = torch.tensor(rows, device="cuda")
        want = oracle.gemm_bf16(_bits(a[idx]), _bits(b))
        want32 = torch.from_numpy(want.copy()).view(torch.bfloat16).float().numpy()
        got = out[0][idx].cpu().float().numpy()
        ref32 = (a[idx].float() @ b.float()).cpu().numpy()           # f32 reference of the rounded operands
        res["parity"] = _parity(tol=1e-2, rel_fro=float(np.linalg.norm(got - ref32) / np.linalg.norm(ref32)),
                                rel_fro_vs_checker=float(np.linalg.norm(got - want32) / np.linalg.norm(want32)),
                                sample="first and last 32 rows of C (all 4096 columns) of the last timed launch against an "
                                       "f32 product of the rounded operands and against the scalar C restatement")
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


def wl_gemm_fp8(torch, tyr, steps, warmup, cpu, parity):
    M = N = K = 8192
    torch.manual_seed(3)
    aq, sa = tyr.quantize_e4m3(_normal(torch, M, K))
    bq, sb = tyr.quantize_e4m3(_normal(torch, K, N))
    out = [None]

    def fn():
        out[0] = tyr.gemm_fp8(aq, bq, sa, sb)
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    res = {
        "metric": "GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "fp8_e4m3",
        "config": {"workload": "fp8 e4m3 GEMM M=N=K=8192, per-tensor f32 scales, bf16 out"},
        "roofline": _mfma_roofline(torch, "mfma_fp8", "gemm_fp8_fast_kernel<false>", tf, TRAFFIC["gemm_fp8"]),
    }
    if parity:
        import numpy as np
        import oracle
        rows = list(range(0, 16)) + list(range(M - 16, M))
        idx = torch.tensor(rows, device="cuda")
        _, want = oracle.gemm_fp8(aq[idx].cpu().view(torch.uint8).numpy(), bq.cpu().view(torch.uint8).numpy(), sa, sb)
        got = out[0][idx].cpu().float().numpy()
        res["parity"] = _parity(tol=1e-2, rel_fro=float(np.linalg.norm(got - want) / np.linalg.norm(want)),
                                sample="first and last 16 rows of C (all 8192 columns) of the last timed launch against the "
                                       "f32 product of the dequantised operands (oracle.gemm_fp8)")
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


def _train_setup(torch, tyr, shape, causal, noise):
    """Examples/GPU/RunMhaH100Train.lean:115-146: f32 targets -> bf16 -> target output; noisy f32 master copies."""
    sc = 1.0 / math.sqrt(shape[-1])
    torch.manual_seed(0)
    tq, tk, tv = (torch.randn(*shape).cuda() for _ in range(3))
    target, _ = tyr.flash_attn_fwd(tq.to(torch.bfloat16), tk.to(torch.bfloat16), tv.to(torch.bfloat16), causal=causal, scale=sc)
    init = [t + torch.randn(*shape).cuda() * noise for t in (tq, tk, tv)]
    return sc, target, init


def _train_step_fused(torch, tyr, masters, lows, target, lr, causal, sc):
    """The same step with the element-wise chains as this library's two fused kernels: the bf16 copies of the masters come
    out of the SGD kernel of the previous step, loss and dO out of one pass over O and the target."""
    o, lse = tyr.flash_attn_fwd(lows[0], lows[1], lows[2], causal=causal, scale=sc)
    loss, d_o = tyr.mse_loss_grad(o, target)
    grads = tyr.flash_attn_bwd(lows[0], lows[1], lows[2], o, lse, d_o, causal=causal, scale=sc)
    new_m, new_l = [], []
    for m, g in zip(masters, grads):
        a, b = tyr.sgd_step(m, g, lr, in_place=True)
        new_m.append(a)
        new_l.append(b)
    return new_m, new_l, loss


def _train_step(torch, tyr, qM, kM, vM, target, lr, causal, sc):
    """oneKernelTrainStep (Examples/GPU/RunMhaH100Train.lean:77-93): cast the f32 masters to bf16, forward, loss =
    0.5 mean((O - target)^2), dO = (O - target) / numel in bf16, backward, SGD on the masters.  The casts, the loss and the
    update are LibTorch elementwise calls in the reference too; forward and backward are this library's kernels."""
    q, k, v = qM.to(torch.bfloat16), kM.to(torch.bfloat16), vM.to(torch.bfloat16)
    o, lse = tyr.flash_attn_fwd(q, k, v, causal=causal, scale=sc)
    diff = o.float() - target.float()
    loss = (diff * diff).mean() * 0.5
    d_o = (diff / diff.numel()).to(torch.bfloat16)
    dq, dk, dv = tyr.flash_attn_bwd(q, k, v, o, lse, d_o, causal=causal, scale=sc)
    return qM - dq.float() * lr, kM - dk.float() * lr, vM - dv.float() * lr, loss


def _wl_train(torch, tyr, steps, warmup, cpu, parity, shape, causal, lr, label):
    B, H, N, D = shape
    sc, target, init = _train_setup(torch, tyr, shape, causal, 0.5)
    state = [t.clone() for t in init]
    losses = []

    def fn_torch_elementwise():
        q, k, v, loss = _train_step(torch, tyr, state[0], state[1], state[2], target, lr, causal, sc)
        state[0], state[1], state[2] = q, k, v
        losses.append(loss)
    # The same step with LibTorch element-wise calls around the kernels is a comparison leg: it runs with the output check
    # only, so that a profile taken with --no-parity holds the kernels of the fused step and nothing else.
    ms_torch_elementwise = time_steps(torch, fn_torch_elementwise, max(5, steps // 3), 2)[1] if parity else None
    fstate = {"m": [t.clone() for t in init]}
    fstate["l"] = [t.to(torch.bfloat16) for t in fstate["m"]]

    def fn():
        fstate["m"], fstate["l"], loss = _train_step_fused(torch, tyr, fstate["m"], fstate["l"], target, lr, causal, sc)
        losses.append(loss)
    wall, ms = time_steps(torch, fn, steps, warmup)
    flop = 14.0 * B * H * N * N * D / (2.0 if causal else 1.0)
    tf = flop / (ms * 1e-3) / 1e12
    res = {
        "metric": "train step TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
        "dtype": "bf16 kernels, f32 master weights",
        "config": {"workload": f"attention train step ({label}): cast + forward + MSE loss + backward + SGD, "
                               f"B={B} H={H} N={N} D={D}, {'causal' if causal else 'non-causal'}; element-wise chains fused "
                               f"(tyr_hip_mse_loss_grad, tyr_hip_sgd_step)",
                   "ms_per_step_with_libtorch_elementwise": ms_torch_elementwise,
                   "flop_convention": "forward 4 + backward 10 = 14*B*H*N^2*D" + ("/2 (causal half)" if causal else ""),
                   "kernel_ms_per_step": ms, "kernel_steps_per_sec": 1e3 / ms, "lr": lr},
        "roofline": _mfma_roofline(torch, "mfma_bf16", "flash_attn_fwd_kernel + " + BWD_KERNELS + " + mse_grad_kernel + sgd_kernel",
                                   tf, None),
    }
    if parity:
        # fresh run of 12 steps from the initial state: the loss must fall (the reference's `ok`), and one step's updated
        # masters must match a float64 step computed by the CPU checker on the same bf16-rounded q, k, v
        import numpy as np
        import oracle
        st = [t.clone() for t in init]
        fm = [t.clone() for t in init]
        fl = [t.to(torch.bfloat16) for t in fm]
        ls, same = [], True
        for _ in range(12):
            st[0], st[1], st[2], loss = _train_step(torch, tyr, st[0], st[1], st[2], target, lr, causal, sc)
            fm, fl, floss = _train_step_fused(torch, tyr, fm, fl, target, lr, causal, sc)
            # the fused element-wise kernels reproduce the LibTorch chain bit for bit, so both runs stay identical
            same = same and all(bool(torch.equal(a, b)) for a, b in zip(st, fm)) and \
                abs(float(loss) - float(floss)) <= 1e-5 * abs(float(loss))
            ls.append(float(loss))
        b, h = B - 1, H - 1
        qb, kb, vb = (t.to(torch.bfloat16) for t in init)
        sl = lambda t: _bits(t[b:b + 1, h:h + 1])
        o, lse = tyr.flash_attn_fwd(qb, kb, vb, causal=causal, scale=sc)
        diff = o.float() - target.float()
        d_o = (diff / diff.numel()).to(torch.bfloat16)
        want = oracle.attn_bwd_f64(sl(qb), sl(kb), sl(vb), sl(d_o), causal, sc)
        got = tyr.flash_attn_bwd(qb, kb, vb, o, lse, d_o, causal=causal, scale=sc)
        rel = max(float(np.linalg.norm(g_[b, h].cpu().float().numpy() - w_[0, 0]) / max(np.linalg.norm(w_[0, 0]), 1e-30))
                  for g_, w_ in zip(got, want))
        res["parity"] = _parity(tol=1e-2, rel_fro=rel, ok=rel <= 1e-2 and ls[-1] < ls[0] and same, init_loss=ls[0], final_loss=ls[-1],
                                fused_equals_libtorch_chain=float(same),
                                sample=f"12 steps from the initial state, once with LibTorch element-wise calls and once with the fused "
                                       f"kernels (masters must stay bit-identical; loss must fall, as the reference's runner demands); "
                                       f"dQ, dK, dV of the first step, head ({b},{h}), against oracle.attn_bwd_f64")
    if cpu:
        from oracle import libtorch_path as lt
        hs = min(H, 4)
        qc, kc, vc = (t[:1, :hs].cpu().clone() for t in init)
        tgt = target[:1, :hs].float().cpu()
        lt.train_step(qc[:, :1], kc[:, :1], vc[:, :1], tgt[:, :1], lr, causal)
        reps, t0 = 0, time.perf_counter()
        while reps < 2 or (time.perf_counter() - t0 < 8 and reps < 200):
            lt.train_step(qc, kc, vc, tgt, lr, causal)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        torch_ms_full = dt * 1e3 * (B * H) / hs
        res["cpu_baseline"] = {"value": flop * hs / (B * H) / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "port",
                               "sample": f"LibTorch CPU oneTorchTrainStep (f32 SDPA + autograd + SGD) on {hs} of {B * H} heads, "
                                         f"{reps} reps, {dt * 1e3:.1f} ms each",
                               "torch_ms_per_step_scaled_to_all_heads": torch_ms_full,
                               "kernel_speedup_vs_torch": torch_ms_full / ms}
    return res


def wl_train_step(torch, tyr, steps, warmup, cpu, parity):
    return _wl_train(torch, tyr, steps, warmup, cpu, parity, (16, 16, 4096, 128), True, 200.0, "benchmark shape")


def wl_train_step_ref_shape(torch, tyr, steps, warmup, cpu, parity):
    return _wl_train(torch, tyr, steps, warmup, cpu, parity, (1, 1, 128, 64), False, 200.0,
                     "the shape of Examples/GPU/RunMhaH100Train.lean")


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


def wl_rope(torch, tyr, steps, warmup, cpu, parity):
    B, S, H, D = 16, 4096, 16, 128
    torch.manual_seed(0)
    x0 = torch.randn(B, S, H, D).to(torch.bfloat16).cuda()
    xs = [x0] + [torch.randn(B, S, H, D, device="cuda").to(torch.bfloat16) for _ in range(2)]   # 268 MB each, rotated
    cos, sin = _rotary_table(torch, S, D)
    it = [0]

    def fn():
        it[0] += 1
        return tyr.rope_fwd(xs[it[0] % 3], cos, sin)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 2 * B * S * H * D * 2 + 2 * S * (D // 2) * 4
    res = _hbm_result("rotary GB/s", "rotary embedding, bf16 [16,4096,16,128], cos/sin f32 [4096,64]",
                      "rope_kernel<bf16>", nbytes, ms, wall, "f32 arithmetic on bf16 data")
    if parity:
        import numpy as np
        import oracle
        y = tyr.rope_fwd(x0, cos, sin)
        want = oracle.rope(_bits(x0[B - 1:]), cos.cpu().numpy(), sin.cpu().numpy())
        bad = int((_bits(y[B - 1:]) != want).sum())
        res["parity"] = {"mismatching_elements": bad, "tol": 0, "ok": bad == 0,
                         "sample": "last batch entry (4096 x 16 x 128), bit for bit against oracle.rope"}
    if cpu:
        from oracle import libtorch_path as lt
        xc = xs[0][:1].cpu()
        dt, reps = _cpu_time(lambda: lt.apply_rotary_emb(xc, cos.cpu(), sin.cpu()))
        res["cpu_baseline"] = {"value": nbytes / B / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU slice/mul/sub/cat sequence on 1 of 16 batch entries, {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def _rotary_table(torch, seq_len, head_dim, base=10000.0):
    """(cos, sin) f32 [seq_len, head_dim/2] on the device: cos / sin of t * base^(-2i/D), the table of
    `compute_rotary_freqs_impl` (cc/src/tyr.cpp:3801-3835)."""
    inv = 1.0 / torch.pow(base, torch.arange(0, head_dim, 2, dtype=torch.float32) / float(head_dim))
    fr = torch.outer(torch.arange(seq_len, dtype=torch.float32), inv)
    return torch.cos(fr).cuda(), torch.sin(fr).cuda()


def wl_layernorm(torch, tyr, steps, warmup, cpu, parity):
    rows, d = 65536, 1024
    torch.manual_seed(0)
    x0, r0 = (torch.rand(rows, d).to(torch.bfloat16).cuda() for _ in range(2))
    xs = [(x0, r0)] + [(torch.rand(rows, d, device="cuda").to(torch.bfloat16), torch.rand(rows, d, device="cuda").to(torch.bfloat16))
                       for _ in range(2)]
    w, b = torch.rand(d).to(torch.bfloat16).cuda(), torch.rand(d).to(torch.bfloat16).cuda()
    it = [0]

    def fn():
        it[0] += 1
        x, r = xs[it[0] % 3]
        return tyr.layernorm_residual(x, r, w, b, 1e-5)
    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = 4 * rows * d * 2 + 2 * d * 2
    res = _hbm_result("layernorm GB/s", "fused residual + LayerNorm, bf16, 65536 rows of 1024",
                      "layernorm_residual_kernel<2>", nbytes, ms, wall, "f32 arithmetic on bf16 data")
    if parity:
        import numpy as np
        import oracle
        out, resid = tyr.layernorm_residual(x0, r0, w, b, 1e-5)
        sl = slice(rows - 512, rows)
        wo, wr = oracle.layernorm_residual(_bits(x0[sl]), _bits(r0[sl]), _bits(w), _bits(b), 1e-5)
        bad = int((_bits(resid[sl]) != wr).sum())
        wo32 = torch.from_numpy(wo.copy()).view(torch.bfloat16).float().numpy()
        err = float(np.abs(out[sl].cpu().float().numpy() - wo32).max())
        tol = 5e-3 + 2 ** -7 * 4
        res["parity"] = {"max_abs": err, "residual_mismatching_elements": bad, "tol": tol, "ok": bad == 0 and err <= tol,
                         "sample": "last 512 rows: residual sum bit for bit, normalised output within one bf16 ulp of the "
                                   "float64 checker (oracle.layernorm_residual)"}
    if cpu:
        from oracle import libtorch_path as lt
        xc, rc = (t.cpu() for t in xs[0])            # all rows: a slice that fits the host caches would flatter the CPU
        wc, bc = w.cpu(), b.cpu()
        dt, reps = _cpu_time(lambda: lt.layer_norm_residual(xc, rc, wc, bc, 1e-5))
        res["cpu_baseline"] = {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU add + layer_norm on all 65536 rows, {reps} reps, {dt * 1e3:.1f} ms each"}
    return res


def wl_copy_kernel(torch, tyr, steps, warmup, cpu, parity):
    n = 1 << 30
    srcs = [torch.empty(n, dtype=torch.uint8, device="cuda").random_() for _ in range(2)]
    it = [0]
    out = [None]

    def fn():
        it[0] += 1
        out[0] = tyr.copy(srcs[it[0] % 2])
    wall, ms = time_steps(torch, fn, steps, warmup)
    res = _hbm_result("copy GB/s", "device copy kernel, 1 GiB", "copy_kernel", 2 * n, ms, wall, "u8")
    if parity:
        same = bool(torch.equal(out[0], srcs[it[0] % 2]))
        res["parity"] = {"identical": same, "tol": 0, "ok": same, "sample": "all 2^30 bytes of the last timed launch against its source"}
    if cpu:
        sc = srcs[0][: n // 8].cpu()
        dt, reps = _cpu_time(lambda: sc.clone())
        res["cpu_baseline"] = {"value": 2 * (n // 8) / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"LibTorch CPU clone of 128 MiB, {reps} reps, {dt * 1e3:.0f} ms each"}
    return res


def wl_decode_step(torch, tyr, steps, warmup, cpu, parity):
    """The decode step's cache update followed by attention over the cache (forwardStep order)."""
    B, Hq, Hkv, L, D = 32, 32, 8, 8192, 128
    torch.manual_seed(1)
    q = torch.randn(B, Hq, 1, D).to(torch.bfloat16).cuda()
    kn, vn = (torch.randn(B, Hkv, 1, D).to(torch.bfloat16).cuda() for _ in range(2))
    caches = _decode_caches(torch, B, Hkv, L, D, 4)
    cos_t, sin_t = _rotary_table(torch, L, D)
    cos, sin = cos_t[L - 1:].contiguous(), sin_t[L - 1:].contiguous()
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
    if parity:
        import numpy as np
        import oracle
        k, v = caches[0]
        qr = tyr.decode_rope_append(q, kn, vn, cos, sin, k, v, L - 1)
        o, lse = tyr.gqa_decode(qr, k, v, scale=sc, kv_len=L)
        c_, s_ = cos.cpu().numpy(), sin.cpu().numpy()
        want_q = oracle.rope(_bits(q.view(B, 1, Hq, D)), c_, s_).reshape(B, Hq, 1, D)
        want_k = oracle.rope(_bits(kn.view(B, 1, Hkv, D)), c_, s_).reshape(B, Hkv, D)
        bad = int((_bits(qr) != want_q).sum()) + int((_bits(k[:, :, L - 1]) != want_k).sum()) + \
            int((~torch.eq(v[:, :, L - 1], vn[:, :, 0])).sum())
        b = B - 1
        wo, wl = oracle.gqa_decode(_bits(qr[b:b + 1]), _bits(k[b:b + 1]), _bits(v[b:b + 1]), sc, 1)
        wo32 = torch.from_numpy(wo.copy()).view(torch.bfloat16).float().numpy()
        err = float(np.abs(o[b:b + 1].cpu().float().numpy() - wo32).max())
        res["parity"] = {"max_abs_o": err, "append_mismatching_elements": bad, "tol": 2e-2, "ok": bad == 0 and err <= 2e-2,
                         "sample": "rotated q, appended k and v rows bit for bit (oracle.rope); attention of the last sequence "
                                   "against oracle.gqa_decode"}
    return res


def wl_copy(torch, tyr, steps, warmup, cpu, parity):
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


def _wl_mfma_sustain(torch, kind):
    sp = sustained_peak(torch, kind)
    tf = sp["value"]
    return {"metric": "sustained MFMA TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": 0.0, "wall_ms_per_step": 0.0,
            "dtype": "bf16" if kind == "mfma_bf16" else "fp8_e4m3",
            "config": {"workload": "MFMA-only loop on normally distributed operands (ceiling calibration): " + sp["how"]},
            "roofline": {"bound": "mfma", "kernel": "mfma_sustain_kernel", "achieved": tf, "peak": PEAK[kind],
                         "unit": "TFLOP/s", "frac": tf / PEAK[kind], "traffic": 0}}


def wl_mfma_bf16(torch, tyr, steps, warmup, cpu, parity):
    return _wl_mfma_sustain(torch, "mfma_bf16")


def wl_mfma_fp8(torch, tyr, steps, warmup, cpu, parity):
    return _wl_mfma_sustain(torch, "mfma_fp8")


def wl_dsl_simple_gemm(torch, tyr, steps, warmup, cpu, parity):
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
    res = {"metric": "emitted GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
           "dtype": "bf16",
           "config": {"workload": "tile-DSL program simpleGemm emitted for gfx950, bf16 x bf16 -> f32, M=N=8192 K=512, "
                                  "64x64 tile per one-wave workgroup"},
           "roofline": _mfma_roofline(torch, "mfma_bf16", "simpleGemm (emitted)", tf, TRAFFIC.get("dsl_simple_gemm"))}
    if parity:
        ref = a[:128].float() @ b.float()
        rel = float((c[:128] - ref).norm() / ref.norm())
        res["parity"] = _parity(tol=1e-2, rel_fro=rel, sample="first 128 rows of C against an f32 product of the rounded operands")
    return res


def wl_dsl_h100_gemm(torch, tyr, steps, warmup, cpu, parity):
    """The reference's H100 bf16 GEMM surface (Tyr/GPU/Kernels/Bf16Gemm.lean:64-73: 128x256 output tile, four K slices
    of 64, B as N x K) emitted for gfx950: a group of four waves per tile, B read from LDS by the products."""
    from tyr_amd.dsl import kernels, runtime
    M = N = 8192
    K = 256                                                     # fixed by the program
    torch.manual_seed(0)
    a = (_normal(torch, M, K) * K ** -0.25).to(torch.bfloat16)
    b = (_normal(torch, N, K) * K ** -0.25).to(torch.bfloat16)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    kern = kernels.tkH100Bf16GemmFwd()
    fn = lambda: runtime.launch(kern, [a, b, c, M, N, K], grid=(N // 256, M // 128, 1), block=(128, 1, 1))
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    nbytes = (M * K + N * K + M * N) * 2
    res = {"metric": "emitted GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
           "dtype": "bf16",
           "config": {"workload": "tile-DSL program tkH100Bf16GemmFwd emitted for gfx950, bf16 x bf16 -> bf16, M=N=8192 K=256 "
                                  "(K is fixed by the program), 128x256 tile per group of four waves",
                      "note": f"at K = 256 the problem moves {nbytes:,} B for 34.4 GFLOP: {nbytes / (ms * 1e-3) / 1e9:.0f} GB/s"},
           "roofline": _mfma_roofline(torch, "mfma_bf16", "tkH100Bf16GemmFwd (emitted)", tf, TRAFFIC["dsl_h100_gemm"])}
    if parity:
        ref = a[:256].float() @ b.float().t()
        rel = float((c[:256].float() - ref).norm() / ref.norm())
        res["parity"] = _parity(tol=1e-2, rel_fro=rel, sample="first 256 rows of C against an f32 product of the rounded operands")
    return res


def wl_dsl_lcf_attn(torch, tyr, steps, warmup, cpu, parity):
    """The reference's load-compute-finish attention surface for D = 128 (Tyr/GPU/Kernels/MhaH100LCF.lean:29-82,109-132: one
    64-row query tile per block, 24 KV tiles of 128 rows, i.e. sequence length 3072, non-causal, scale 1/sqrt(128)) emitted
    for gfx950: a group of two waves per query tile, K and V read from LDS by the products.  The program addresses one
    [3072, 128] head at column block blockIdx.x, so the heads are laid side by side ([sequence, heads * 128]) and the grid
    is (heads, 3072 / 64)."""
    from tyr_amd.dsl import kernels, runtime
    H, S, D = 64, 3072, 128
    torch.manual_seed(0)
    q, k, v = (_normal(torch, S, H * D).to(torch.bfloat16) for _ in range(3))
    o = torch.zeros(S, H * D, dtype=torch.bfloat16, device="cuda")
    kern = kernels.tkMhaH100LCFFwd128()
    fn = lambda: runtime.launch(kern, [q, k, v, o, S, D], grid=(H, S // 64, 1), block=(64, 1, 1))   # 2 warps of the reference
    wall, ms = time_steps(torch, fn, steps, warmup)
    tf = 4.0 * H * S * S * D / (ms * 1e-3) / 1e12
    res = {"metric": "emitted attention TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "wall_ms_per_step": wall,
           "dtype": "bf16",
           "config": {"workload": "tile-DSL program tkMhaH100LCFFwd128 emitted for gfx950: non-causal attention forward, bf16, "
                                  "64 heads side by side, N=3072 (24 KV tiles of 128), D=128, 64 query rows per two-wave group",
                      "flop_convention": "4*H*N^2*D (non-causal)"},
           "roofline": _mfma_roofline(torch, "mfma_bf16", "tkMhaH100LCFFwd128 (emitted)", tf, TRAFFIC.get("dsl_lcf_attn"))}
    if parity:
        import numpy as np
        import oracle
        e_o = 0.0
        heads = (0, H - 1)
        for h in heads:
            sl = lambda t: _bits(t[:, h * D:(h + 1) * D].contiguous().view(1, 1, S, D))
            o64, _ = oracle.attn_fwd_f64(sl(q), sl(k), sl(v), False, 0.08838834764)
            e_o = max(e_o, float(np.abs(o[:, h * D:(h + 1) * D].cpu().float().numpy() - o64[0, 0]).max()))
        res["parity"] = _parity(tol=2e-2, max_abs_o=e_o,
                                sample=f"heads {list(heads)}, all 3072 rows, against the float64 checker (oracle.attn_fwd_f64)")
    return res


WORKLOADS = {"attn_fwd_causal": wl_attn, "attn_bwd_causal": wl_attn_bwd, "mha_train_step": wl_train_step,
             "mha_train_step_ref_shape": wl_train_step_ref_shape, "gqa_decode": wl_decode, "gqa_decode_split4": wl_decode_split4,
             "gqa_decode_small_batch": wl_decode_small_batch, "gemm_bf16": wl_gemm_bf16,
             "gemm_fp8": wl_gemm_fp8, "decode_step": wl_decode_step, "rope_fwd": wl_rope, "layernorm_residual": wl_layernorm,
             "copy_kernel": wl_copy_kernel, "dsl_simple_gemm": wl_dsl_simple_gemm, "dsl_h100_gemm": wl_dsl_h100_gemm,
             "dsl_lcf_attn": wl_dsl_lcf_attn}
CALIBRATION = {"copy_1gib": wl_copy, "mfma_sustain_bf16": wl_mfma_bf16, "mfma_sustain_fp8": wl_mfma_fp8}


# the configurations of the benchmark that run on the GPU (configuration 1 is the LibTorch-CPU plumbing case)
BASELINE_CONFIGS = {"cfg2_gemm_bf16_4096": "gemm_bf16", "cfg3_attn_fwd_causal_b16_h16_n4096_d128": "attn_fwd_causal",
                    "cfg4_gqa_decode_b32_hq32_hkv8_l8192": "gqa_decode", "cfg5_gemm_fp8_8192": "gemm_fp8"}


def _summary(r):
    """The few figures of a workload record that the one-line output carries."""
    if "error" in r:
        return {"workload": r["workload"], "error": r["error"][:200]}
    roof, par, cpu = r.get("roofline") or {}, r.get("parity") or {}, r.get("cpu_baseline") or {}
    d = {"workload": r["workload"], "ms_per_step": round(r["ms_per_step"], 5), "value": round(r["value"], 1), "unit": r["unit"],
         "bound": roof.get("bound"), "frac": round(roof.get("frac", 0.0), 4), "traffic": roof.get("traffic"),
         "parity_ok": par.get("ok")}
    if "error" in par:
        d["parity_error"] = par["error"][:160]
    if cpu:
        d["cpu_baseline"] = {"value": round(cpu["value"], 4), "unit": cpu["unit"], "cores": cpu["cores"]}
    return d


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="attn_fwd_causal", choices=sorted(WORKLOADS) + sorted(CALIBRATION))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-parity", action="store_true", help="skip the check of the outputs against the CPU checker")
    ap.add_argument("--no-extra", action="store_true", help="measure only --workload")
    ap.add_argument("--details", default=None, metavar="FILE", help="also write the full records (one JSON line) to FILE")
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
    def run(fn, steps, warmup):
        """A failing checker or CPU leg must not take the measurement with it: the workload is then measured again
        without them and the failure is reported in its place."""
        try:
            return fn(torch, tyr_amd, steps, warmup, not args.no_cpu, not args.no_parity)
        except Exception as e:
            if args.no_cpu and args.no_parity:
                raise
            r = fn(torch, tyr_amd, steps, warmup, False, False)
            r["parity"] = {"ok": False, "error": f"checker / CPU leg failed: {type(e).__name__}: {e}"}
            return r

    head = run({**WORKLOADS, **CALIBRATION}[args.workload], args.steps, args.warmup)
    head["workload"] = args.workload
    records = [head]
    if not args.no_extra:
        for name, fn in WORKLOADS.items():
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            try:
                r = run(fn, max(10, args.steps // 2), max(3, args.warmup // 2))
            except Exception as e:                      # a side workload must not take the headline line with it
                r = {"error": f"{type(e).__name__}: {e}"}
            r["workload"] = name
            records.append(r)

    host = {"nproc": os.cpu_count(), "usable_cores": len(os.sched_getaffinity(0)), "torch_threads": torch.get_num_threads()}
    roof = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in head["roofline"].items() if k != "sustained_how"}
    par = head.get("parity")
    line = {
        "metric": head["metric"], "value": round(head["value"], 3), "unit": head["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "settle_ms_before_warmup": PREWARM_MS,
        "ms_per_step": round(head["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic" if DATA == "randn" else "synthetic, every operand 0.5 (power diagnostic, not the benchmark input)",
        "config": head["config"], "roofline": roof,
        "parity": None if par is None else {k: (round(v, 6) if isinstance(v, float) else v) for k, v in par.items() if k != "sample"},
        "cpu_baseline": head.get("cpu_baseline"), "wall_ms_per_step": round(head["wall_ms_per_step"], 5),
        "device": info, "host": host,
    }
    by_name = {r["workload"]: r for r in records}
    line["baseline_configs"] = {label: _summary(by_name[name]) for label, name in BASELINE_CONFIGS.items() if name in by_name}
    if not args.no_extra:
        line["other_workloads"] = [_summary(r) for r in records[1:] if r["workload"] not in BASELINE_CONFIGS.values()]
    details = json.dumps({"details": records, "device": info, "host": host})
    if args.details:
        with open(args.details, "w") as f:
            f.write(details + "\n")
    print(details, file=sys.stderr, flush=True)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
