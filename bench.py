#!/usr/bin/env python3
"""Benchmark of the fused JVP attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

Workload (the headline benchmark configuration): bf16, B=4, H=16, L=4096, D=128, synthetic N(0,1) inputs that
are resident in HBM before the timed region.  A step is one fused dual forward (O and O' in
one kernel).  ``value`` is its throughput in TFLOP/s with the algorithmic FLOP count
12 * B*H*L^2*D (six GEMM-shaped products, 2 FLOPs per multiply-add).  The same JSON line also
carries the causal forward, forward+backward (tangent-path backward, 24 * B*H*L^2*D more) and
the reference's FLOP convention (its tests count 2*(4*B*H*L^2*D + 5*B*H*L^2)) for comparison with
its README, a roofline block for the forward kernel, and the reference's CPU route (math SDPA under
``torch.func.jvp``, fp32) timed on this host on a slab of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak
Z, H, L, D = 4, 16, 4096, 128

# HBM bytes per forward launch.  A recorded constant, not measured in this run: rocprofv3 --pmc
# FETCH_SIZE (x2.0, the factor a plain copy of known size gives) and WRITE_SIZE (x1.0) read 405.4 MB +
# 136.3 MB; the counter runs and their commands are in profiles/fwd3_kernel_bf16_B4_H16_L4096_D128.md.
MEASURED_FWD_TRAFFIC_BYTES = 541.7e6
TRAFFIC_SOURCE = "recorded from the rocprofv3 --pmc runs in profiles/fwd3_kernel_bf16_B4_H16_L4096_D128.md, not measured in this run"


def timed(fn, steps, warmup):
    import torch

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
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall_ms


def cpu_baseline():
    """Reference CPU route (math SDPA under torch.func.jvp, fp32) on this host's cores: one warm-up and three timed
    runs of a bounded sample of the headline workload, the median reported.  The sample is sized for about 5 s per
    run (the whole B*H = 64 heads where the host is fast enough, otherwise as many heads as fit)."""
    import statistics

    import torch

    from oracle import sdpa_jvp

    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    cores = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)

    def run(zb, hb):
        q, k, v, qt, kt, vt = [torch.randn(zb, hb, L, D, generator=g) for _ in range(6)]
        t0 = time.perf_counter()
        sdpa_jvp.forward(q, k, v, qt, kt, vt)
        return time.perf_counter() - t0

    run(1, 1)  # pages in the libraries
    t2 = run(1, 2)
    heads = int(min(Z * H, max(2, 5.0 / max(t2 / 2, 1e-3))))
    zb, hb = (1, heads) if heads <= H else (heads // H, H)
    run(zb, hb)  # warm-up at the sample's size
    runs = sorted(run(zb, hb) for _ in range(3))
    dt = statistics.median(runs)
    flops = 12.0 * zb * hb * L * L * D
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"math SDPA + torch.func.jvp fp32 dual forward on B={zb},H={hb},L={L},D={D}: 1 warm-up + 3 runs, median "
                  f"{dt:.2f} s (min {runs[0]:.2f}, max {runs[-1]:.2f})"
                  + ("; the whole headline shape" if zb * hb == Z * H
                     else f"; {zb * hb} of {Z * H} heads, the whole shape would take ~{dt * Z * H / (zb * hb):.0f} s"),
    }


def hvp_sweep(be, _lib):
    """benchmark configuration 5: bf16 B1 H16 D128 causal, L swept; fused dual forward + the backward of
    sum(O' * gO') w.r.t. q, k, v (the Hessian-vector-product pattern): time and peak HBM vs L."""
    import torch

    dev = torch.device("cuda:0")
    rows = []
    for Ls in (1024, 4096, 16384, 32768):
        torch.cuda.empty_cache()
        g = torch.Generator(device=dev).manual_seed(Ls)
        q, k, v, qt, kt, vt, gt = [
            torch.randn(1, 16, Ls, 128, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(7)
        ]
        scale = 128**-0.5

        def step():
            o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, True, scale)
            return be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, None, gt, None, _lib.MASK_NONE, True, scale)

        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        ms, _ = timed(step, 3, 1)
        peak = torch.cuda.max_memory_allocated() - base
        n = 16.0 * Ls * Ls * 128
        rows.append({"L": Ls, "ms": ms, "tflops": (12 + 24) * n / 2 / (ms * 1e-3) / 1e12,
                     "peak_extra_hbm_mb": peak / 2**20, "inputs_mb": 7 * q.numel() * 2 / 2**20,
                     "one_fp32_score_tensor_mb_if_materialised": 16.0 * Ls * Ls * 4 / 2**20})
    return rows


def shape_rows(be, _lib):
    """Shapes next to the headline one, no mask: the other benchmark configurations' shapes, D = 32 and
    D = 256 (the smallest and the largest head dim the reference admits), 16 query heads over 4 key/value heads, and 4096 queries over 512 keys (the last two are
    shapes the reference refuses), fp32 at D = 256, and the headline shape with dropout; then benchmark configurations 3 and 4 with their masks
    (causal; key padding; additive bias).  Dual forward and dual backward, counted as 12 and 24 flops per (query, key, d) triple."""
    import torch

    dev = torch.device("cuda:0")
    rows = {}
    for name, (Zs, Hs, Hk, Lq, Lk, Ds, dtype, *drop) in {
        "bf16_B4_H16_L2048_D32": (4, 16, 16, 2048, 2048, 32, torch.bfloat16),
        "bf16_B4_H16_L2048_D64_config2": (4, 16, 16, 2048, 2048, 64, torch.bfloat16),
        "bf16_B4_H16_L2048_D256": (4, 16, 16, 2048, 2048, 256, torch.bfloat16),
        "fp16_B2_H32_L4096_D128_config3_noncausal": (2, 32, 32, 4096, 4096, 128, torch.float16),
        "fp32_B4_H8_L1024_D64_config4_nomask": (4, 8, 8, 1024, 1024, 64, torch.float32),
        "bf16_B4_H16_over_4_kv_heads_L4096_D128": (4, 16, 4, 4096, 4096, 128, torch.bfloat16),
        "bf16_B4_H16_Lq4096_Lk512_D128": (4, 16, 16, 4096, 512, 128, torch.bfloat16),
        "fp32_B4_H8_L1024_D256": (4, 8, 8, 1024, 1024, 256, torch.float32),
        "bf16_B4_H16_L4096_D128_dropout_0.1": (4, 16, 16, 4096, 4096, 128, torch.bfloat16, 0.1),
    }.items():
        dp = drop[0] if drop else 0.0
        g = torch.Generator(device=dev).manual_seed(11)
        mk = lambda h, l: torch.randn(Zs, h, l, Ds, generator=g, device=dev).to(dtype)  # noqa: E731
        q, qt, go, gt = [mk(Hs, Lq) for _ in range(4)]
        k, v, kt, vt = [mk(Hk, Lk) for _ in range(4)]
        scale = Ds**-0.5
        ms_f, _ = timed(lambda: be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, False, scale, dp, 7), 20, 12)
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, False, scale, dp, 7)
        ms_b, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, False, scale,
                                       dropout_p=dp, dropout_seed=7), 10, 6)
        n = float(Zs) * Hs * Lq * Lk * Ds
        rows[name] = {"fwd_ms": ms_f, "fwd_tflops": 12 * n / (ms_f * 1e-3) / 1e12,
                      "bwd_ms": ms_b, "bwd_tflops": 24 * n / (ms_b * 1e-3) / 1e12}
    # the benchmark configurations that come with a mask, as they are specified: flops counted over the attended
    # (query, key) pairs only
    for name, (Zs, Hs, Ls, Ds, dtype, mode) in {
        "fp16_B2_H32_L4096_D128_config3_causal": (2, 32, 4096, 128, torch.float16, "causal"),
        "fp32_B4_H8_L1024_D64_config4a_key_padding": (4, 8, 1024, 64, torch.float32, "keypad"),
        "fp32_B4_H8_L1024_D64_config4b_additive_bias": (4, 8, 1024, 64, torch.float32, "bias"),
    }.items():
        g = torch.Generator(device=dev).manual_seed(13)
        q, k, v, qt, kt, vt, go, gt = [torch.randn(Zs, Hs, Ls, Ds, generator=g, device=dev).to(dtype) for _ in range(8)]
        mask, kind, causal, frac = None, _lib.MASK_NONE, False, 1.0
        if mode == "causal":
            causal, frac = True, (Ls + 1) / (2.0 * Ls)
        elif mode == "keypad":  # valid length per batch entry uniform in [L/2, L]
            lens = torch.randint(Ls // 2, Ls + 1, (Zs,), generator=g, device=dev)
            mask, kind = (torch.arange(Ls, device=dev)[None, :] < lens[:, None]).view(Zs, 1, 1, Ls), _lib.MASK_BOOL
            frac = lens.float().mean().item() / Ls
        else:
            mask, kind = torch.randn(Zs, Hs, Ls, Ls, generator=g, device=dev).to(dtype), _lib.MASK_ADD
        scale = Ds**-0.5
        ms_f, _ = timed(lambda: be.fwd(q, k, v, qt, kt, vt, mask, kind, causal, scale), 20, 12)
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, mask, kind, causal, scale)
        ms_b, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, mask, kind, causal, scale), 10, 6)
        n = float(Zs) * Hs * Ls * Ls * Ds * frac
        rows[name] = {"attended_fraction": frac, "fwd_ms": ms_f, "fwd_tflops": 12 * n / (ms_f * 1e-3) / 1e12,
                      "bwd_ms": ms_b, "bwd_tflops": 24 * n / (ms_b * 1e-3) / 1e12}
    return rows


def mask_rows(be, _lib, q, k, v, qt, kt, vt, go, gt, scale):
    """The headline shape with explicit masks: dual forward / backward times for a dense random boolean
    mask (nothing to skip), a block-diagonal mask of four segments and a band of +-256 keys (tiles
    without an attended entry are skipped through the tile lists), the time of the scan that makes
    the lists (an HBM-bound pass: it reads the mask once per list), and an additive mask shared by the heads."""
    import torch

    dev = q.device
    g = torch.Generator(device=dev).manual_seed(7)
    idx = torch.arange(L, device=dev)
    seg = (idx * 4) // L
    masks = {
        "dense_bool_ZHLL": torch.rand(Z, H, L, L, generator=g, device=dev) > 0.1,
        "block_diagonal_x4_Z1LL": (seg[:, None] == seg[None, :]).view(1, 1, L, L).expand(Z, 1, L, L).contiguous(),
        "band_256_11LL": ((idx[:, None] - idx[None, :]).abs() <= 256).view(1, 1, L, L),
    }
    rows = {}
    for name, m in masks.items():
        ms_f, _ = timed(lambda: be.fwd(q, k, v, qt, kt, vt, m, _lib.MASK_BOOL, False, scale), 20, 12)
        o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, m, _lib.MASK_BOOL, False, scale)
        ms_b, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, m, _lib.MASK_BOOL, False, scale), 10, 6)

        def scan():
            if hasattr(m, "_jvpfa_tiles"):
                del m._jvpfa_tiles
            _lib.tile_lists(q, m, _lib.MASK_BOOL, True)

        ms_s, _ = timed(scan, 10, 6)
        rows[name] = {"attended_fraction": m.float().mean().item(), "fwd_ms": ms_f, "bwd_ms": ms_b, "scan_ms": ms_s,
                      "scan_GBps": 2.0 * m.numel() / (ms_s * 1e-3) / 1e9}
        del m
    # an additive mask (a bias shared by the heads): dual forward / backward and the backward without tangents
    bias = torch.randn(Z, 1, L, L, generator=g, device=dev).to(q.dtype)
    ms_f, _ = timed(lambda: be.fwd(q, k, v, qt, kt, vt, bias, _lib.MASK_ADD, False, scale), 20, 12)
    o, ot, M, mu = be.fwd(q, k, v, qt, kt, vt, bias, _lib.MASK_ADD, False, scale)
    ms_b, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, bias, _lib.MASK_ADD, False, scale), 10, 6)
    ms_p, _ = timed(lambda: be.bwd(q, k, v, None, None, None, o, None, M, None, go, None, bias, _lib.MASK_ADD, False, scale), 10, 6)
    rows["additive_bias_Z1LL"] = {"attended_fraction": 1.0, "fwd_ms": ms_f, "bwd_ms": ms_b, "bwd_without_tangents_ms": ms_p}
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=40,
                    help="untimed launches before the timed ones: the clock of the chip settles over the first 30 or so")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--fwd-only", action="store_true", help="time only the headline forward (for profiling)")
    ap.add_argument("--bwd-only", action="store_true",
                    help="run one forward, then time only the headline backward (for profiling); prints its own line")
    ap.add_argument("--plain-only", action="store_true",
                    help="time the headline shape without tangents (what attention() runs in first-order training): forward, "
                         "then the backward of gO (for profiling); prints its own line")
    ap.add_argument("--masked-fwd-only", action="store_true",
                    help="time the headline dual forward with a dense boolean mask, with an additive mask and with dropout "
                         "0.1 next to the unmasked one (for profiling); prints its own line")
    ap.add_argument("--bwd6-only", action="store_true",
                    help="run one forward, then time the backward that also returns dq', dk', dv' (for profiling)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy, whose known traffic scales the rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings of the forward kernel")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (B*H shards trivially); use --gpus 1")

    import torch

    from jvp_flash_attention_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs an AMD GPU (no CPU path exists)")
    be = _lib.backend()
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    q, k, v, qt, kt, vt, go, gt = [
        torch.randn(Z, H, L, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(8)
    ]
    scale = D**-0.5
    N = float(Z) * H * L * L * D
    fwd_flops, bwd_flops = 12.0 * N, 24.0 * N
    ref_conv_flops = 2.0 * (4.0 * N + 5.0 * Z * H * L * L)

    def fwd(causal=False):
        return be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, causal, scale)

    state = {}

    def fwd_bwd(causal=False):
        o, ot, M, mu = fwd(causal)
        state["g"] = be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, causal, scale)

    if args.bwd_only:
        o, ot, M, mu = fwd()
        ms_b, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, False, scale),
                        args.steps, args.warmup)
        print(json.dumps({"workload": "bf16 B4 H16 L4096 D128 backward of (gO, gT) -> dq, dk, dv", "ms_per_step": ms_b,
                          "tflops_algorithmic": bwd_flops / (ms_b * 1e-3) / 1e12}), flush=True)
        return
    if args.plain_only:
        ms_pf, _ = timed(lambda: be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, scale), args.steps, args.warmup)
        o, _, M, _ = be.fwd(q, k, v, None, None, None, None, _lib.MASK_NONE, False, scale)
        ms_pb, _ = timed(lambda: be.bwd(q, k, v, None, None, None, o, None, M, None, go, None, None, _lib.MASK_NONE, False, scale),
                         args.steps, args.warmup)
        print(json.dumps({"workload": "bf16 B4 H16 L4096 D128 without tangents: forward (4 N flops), backward of gO (10 N)",
                          "fwd_ms": ms_pf, "fwd_tflops": 4.0 * N / (ms_pf * 1e-3) / 1e12,
                          "bwd_ms": ms_pb, "bwd_tflops": 10.0 * N / (ms_pb * 1e-3) / 1e12}), flush=True)
        return
    if args.masked_fwd_only:
        gm = torch.Generator(device=dev).manual_seed(7)
        mb = torch.rand(Z, H, L, L, generator=gm, device=dev) > 0.1
        ma = torch.randn(Z, 1, L, L, generator=gm, device=dev).to(torch.bfloat16)
        row = {"workload": "bf16 B4 H16 L4096 D128 dual forward: no mask | dense boolean mask (Z,H,L,L), 90 % attended | "
                           "additive mask (Z,1,L,L) | dropout 0.1"}
        for name, call in (("none", lambda: fwd()),
                           ("bool", lambda: be.fwd(q, k, v, qt, kt, vt, mb, _lib.MASK_BOOL, False, scale)),
                           ("additive", lambda: be.fwd(q, k, v, qt, kt, vt, ma, _lib.MASK_ADD, False, scale)),
                           ("dropout", lambda: be.fwd(q, k, v, qt, kt, vt, None, _lib.MASK_NONE, False, scale, 0.1, 7))):
            row[name + "_ms"], _ = timed(call, args.steps, args.warmup)
        print(json.dumps(row), flush=True)
        return
    if args.bwd6_only:
        o, ot, M, mu = fwd()
        ms_b6, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, False, scale,
                                        want_tangent_grads=True), args.steps, args.warmup)
        print(json.dumps({"workload": "bf16 B4 H16 L4096 D128 backward of (gO, gT) -> dq, dk, dv, dq', dk', dv'", "ms_per_step": ms_b6,
                          "tflops_algorithmic": bwd_flops * 15 / 12 / (ms_b6 * 1e-3) / 1e12}), flush=True)
        return
    if args.calibrate_copy:
        src = torch.empty(256 * 2**20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    # The secondary rows run first and the headline last: a fresh process needs some thirty launches before the
    # GPU's clock has settled, and the headline is then timed (its own W warm-up launches + K timed ones, as asked
    # for) on a GPU that has been busy for a while, which is the state a training or serving job keeps it in.
    extra = None
    if not args.fwd_only:
        other_shapes = shape_rows(be, _lib)
        masks = mask_rows(be, _lib, q, k, v, qt, kt, vt, go, gt, scale)
        hvp = hvp_sweep(be, _lib)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        ms_fc, _ = timed(lambda: fwd(True), args.steps, args.warmup)
        o, ot, M, mu = fwd()
        ms_b, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, False, scale),
                        max(1, args.steps // 2), 2)
        ms_b6, _ = timed(lambda: be.bwd(q, k, v, qt, kt, vt, o, ot, M, mu, go, gt, None, _lib.MASK_NONE, False, scale,
                                        want_tangent_grads=True), max(1, args.steps // 2), 2)
        del o, ot, M, mu
        ms_fb, _ = timed(fwd_bwd, max(1, args.steps // 2), 2)
        ms_fbc, _ = timed(lambda: fwd_bwd(True), max(1, args.steps // 2), 2)
        peak_mb = torch.cuda.max_memory_allocated() / 2**20
        tf = lambda fl, ms: fl / (ms * 1e-3) / 1e12  # noqa: E731
        extra = {
            "fwd_causal": {"ms": ms_fc, "tflops": tf(fwd_flops / 2, ms_fc),
                           "pct_mfma_peak": 100 * tf(fwd_flops / 2, ms_fc) / PEAK_BF16_TFLOPS},
            "fwd_bwd": {"ms": ms_fb, "tflops": tf(fwd_flops + bwd_flops, ms_fb),
                        "pct_mfma_peak": 100 * tf(fwd_flops + bwd_flops, ms_fb) / PEAK_BF16_TFLOPS},
            "fwd_bwd_causal": {"ms": ms_fbc, "tflops": tf((fwd_flops + bwd_flops) / 2, ms_fbc),
                               "pct_mfma_peak": 100 * tf((fwd_flops + bwd_flops) / 2, ms_fbc) / PEAK_BF16_TFLOPS},
            # the backward alone: pre-pass + bwd2_dkdv (10 products executed) + bwd2_dq (8 executed), 12 counted
            "roofline_backward": {"bound": "mfma", "achieved": tf(bwd_flops, ms_b), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                  "frac": tf(bwd_flops, ms_b) / PEAK_BF16_TFLOPS, "ms": ms_b,
                                  "executed_tflops": tf(bwd_flops * 18 / 12, ms_b),
                                  "kernels": "bwd_prepass + bwd2_dkdv + bwd2_dq <bf16, D=128, dual>"},
            # all six gradients (dq, dk, dv and dq', dk', dv'): 15 products counted
            "bwd_six_gradients": {"ms": ms_b6, "tflops": tf(bwd_flops * 15 / 12, ms_b6),
                                  "pct_mfma_peak": 100 * tf(bwd_flops * 15 / 12, ms_b6) / PEAK_BF16_TFLOPS},
                        "peak_hbm_allocated_mb": peak_mb,
        }
        extra["hvp_sweep_bf16_B1_H16_D128_causal"] = hvp
        extra["masks_bf16_B4_H16_L4096_D128"] = masks
        extra["other_shapes"] = other_shapes
    ms_fwd, wall_fwd = timed(fwd, args.steps, args.warmup)
    out = {
        "metric": "fused JVP dual-forward throughput, bf16 B4 H16 L4096 D128 (non-causal)",
        "value": fwd_flops / (ms_fwd * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_fwd,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,  # the reference publishes no number for this shape or for any AMD GPU
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "bf16 B4 H16 L4096 D128 dual forward (O, O'), no mask, sm_scale=D^-0.5",
                   "flops_per_step": fwd_flops},
        "pct_mfma_peak": 100.0 * fwd_flops / (ms_fwd * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "wall_ms_per_step": wall_fwd,
        "roofline": {
            "bound": "mfma",
            "achieved": fwd_flops / (ms_fwd * 1e-3) / 1e12,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": fwd_flops / (ms_fwd * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
            "traffic": MEASURED_FWD_TRAFFIC_BYTES,
            "traffic_source": TRAFFIC_SOURCE,
            "kernel": "fwd3_kernel<bf16, D=128, dual>",
        },
    }
    if extra is not None:
        extra["fwd_tflops_reference_flop_convention"] = ref_conv_flops / (ms_fwd * 1e-3) / 1e12
        out["extra"] = extra
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
