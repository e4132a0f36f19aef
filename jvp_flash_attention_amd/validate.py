"""Accuracy and speed report for JVP attention on the current GPU.

    python -m jvp_flash_attention_amd.validate --dtype bfloat16 [--seq-lengths 32 64 ... 2048]
                                               [--no-masks] [--no-timing] [--json out.json] [--plots DIR]

Counterpart of the reference's script ``tests/test_jvp_attention.py`` (run as a program there,
README.md:111-113): for every sequence length, mask type (none / boolean / additive) and causal
flag it (1) compares ``JVPAttn.fwd_dual`` under ``fwAD.dual_level()`` and under ``torch.func.jvp``
with PyTorch's math SDPA under forward-mode AD (what the reference's own tests compare with, test file lines 548-617):
primal, tangent, the loss ``mean((out - target)^2)`` and its q/k/v gradients; (2) times the dual
forward the way the reference does (10 warm-up + 100 calls, input clones and ``make_dual``
included, lines 129-143 and 770-780) next to math SDPA; (3) records the peak memory of one call.
After the per-case lines it prints the reference's two tables (summary per case and method, lines 883-937;
time by mask type, lines 940-976) and its speed-up statistics, and writes them with the rows into the JSON
file (lines 1172-1227); with ``--plots DIR`` it also draws the reference's two figures (lines 977-1091): speed-up over
math SDPA and peak memory per sequence length, one panel per (causal, mask) configuration.
Shapes default to the reference's (batch 2, 12 heads, head dim 64, lines 225-230); masks are its
random masks with keep-probability 0.1 (lines 334-394).  TFLOP/s uses the reference's FLOP
convention ``2 * (4 B H L^2 D + 5 B H L^2)``, halved when causal (lines 49-83).
"""
from __future__ import annotations

import argparse
import json
import time
from functools import partial

import torch
import torch.autograd.forward_ad as fwAD
import torch.nn.functional as F
from torch.nn.attention import SDPBackend, sdpa_kernel

from . import MASK_CONST, JVPAttn

TOLERANCE = {"float16": 4e-3, "float32": 2.35e-2, "bfloat16": 3.2e-2}  # reference lines 688-693
DTYPES = {"float16": torch.float16, "float32": torch.float32, "bfloat16": torch.bfloat16}


def flop_count(B, H, L, D, causal):
    f = 2.0 * (4.0 * B * H * L * L * D + 5.0 * B * H * L * L)
    return f / 2 if causal else f


def make_mask(kind, B, H, L, dtype, device):
    if kind == "none":
        return None
    g = torch.Generator(device=device).manual_seed(1042)
    keep = torch.rand(B, H, L, L, generator=g, device=device) > 0.9
    keep[..., 0] |= ~keep.any(-1)  # no fully masked row
    if kind == "boolean":
        return keep
    return torch.where(keep, 0.0, MASK_CONST).to(dtype)


def sdpa_dual(q, k, v, qt, kt, vt, mask, causal):
    sdpa_mask = mask
    if mask is not None and mask.dtype != torch.bool:
        sdpa_mask = mask != MASK_CONST  # the reference's float masks mark masked entries with MASK_CONST
    with sdpa_kernel(SDPBackend.MATH), fwAD.dual_level():
        out = F.scaled_dot_product_attention(fwAD.make_dual(q, qt), fwAD.make_dual(k, kt), fwAD.make_dual(v, vt),
                                             attn_mask=sdpa_mask, is_causal=causal)
        o, ot = fwAD.unpack_dual(out)
        return o.clone(), ot.clone()


def grads_of_mse(fn, q, k, v, target):
    leaves = [x.clone().requires_grad_() for x in (q, k, v)]
    loss = ((fn(*leaves).float() - target.float()) ** 2).mean()
    return loss.detach(), torch.autograd.grad(loss, leaves)


def timed(fn, warmup=10, iters=100):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / iters


def peak_mb(fn):
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    fn()
    torch.cuda.synchronize()
    return (torch.cuda.max_memory_allocated() - base) / 2**20


def run(args):
    dev = torch.device("cuda")
    dtype = DTYPES[args.dtype]
    B, H, D = args.bsz, args.model_dim // args.head_dim, args.head_dim
    rows = []
    for L in args.seq_lengths:
        g = torch.Generator(device=dev).manual_seed(42)
        q, qt, k, kt, v, vt, target = [torch.randn(B, H, L, D, generator=g, device=dev, dtype=dtype) for _ in range(7)]
        for kind in (["none"] if args.no_masks else ["none", "boolean", "additive"]):
            mask = make_mask(kind, B, H, L, dtype, dev)
            for causal in (False, True):
                if causal and kind != "none":
                    continue
                fn = partial(JVPAttn.fwd_dual, attn_mask=mask, causal=causal)
                o_ref, ot_ref = sdpa_dual(q, k, v, qt, kt, vt, mask, causal)
                with fwAD.dual_level():
                    o1, ot1 = (t.clone() for t in fwAD.unpack_dual(fn(fwAD.make_dual(q, qt), fwAD.make_dual(k, kt), fwAD.make_dual(v, vt))))
                o2, ot2 = torch.func.jvp(fn, (q, k, v), (qt, kt, vt))
                sdpa_mask = mask if (mask is None or mask.dtype == torch.bool) else mask != MASK_CONST
                with sdpa_kernel(SDPBackend.MATH):
                    loss_ref, g_ref = grads_of_mse(
                        lambda a, b, c: F.scaled_dot_product_attention(a, b, c, attn_mask=sdpa_mask, is_causal=causal),
                        q, k, v, target)
                loss, g_ours = grads_of_mse(lambda a, b, c: JVPAttn.fwd(a, b, c, attn_mask=mask, causal=causal), q, k, v, target)
                err = lambda a, b: (a.float() - b.float()).abs().max().item()  # noqa: E731
                acc = {
                    "primal": max(err(o1, o_ref), err(o2, o_ref)), "tangent": max(err(ot1, ot_ref), err(ot2, ot_ref)),
                    "loss": abs(loss.item() - loss_ref.item()),
                    "dq": err(g_ours[0], g_ref[0]), "dk": err(g_ours[1], g_ref[1]), "dv": err(g_ours[2], g_ref[2]),
                }
                ok = max(acc["primal"], acc["tangent"]) < TOLERANCE[args.dtype] and max(acc["loss"], acc["dq"], acc["dk"], acc["dv"]) < 5e-4

                def ours():
                    with fwAD.dual_level():
                        return fn(fwAD.make_dual(q.clone(), qt.clone()), fwAD.make_dual(k.clone(), kt.clone()),
                                  fwAD.make_dual(v.clone(), vt.clone()))

                def ours_kernel_only():
                    return JVPAttn.forward(q, k, v, qt, kt, vt, mask, 0.0, causal, None, True, True, False)

                if args.no_timing:  # one call each: the accuracy half of the report only
                    ms, ms_k = timed(ours, 0, 1), timed(ours_kernel_only, 0, 1)
                    ms_sdpa = timed(lambda: sdpa_dual(q, k, v, qt, kt, vt, mask, causal), 0, 1)
                else:
                    ms, ms_k = timed(ours), timed(ours_kernel_only)
                    ms_sdpa = timed(lambda: sdpa_dual(q, k, v, qt, kt, vt, mask, causal), 2, 10)
                fl = 2 * flop_count(B, H, L, D, causal) / 2  # the convention already counts the JVP (x2 inside)
                row = {"L": L, "mask": kind, "causal": causal, "ok": ok, **acc, "ms": ms, "ms_kernel_only": ms_k,
                       "ms_sdpa_math": ms_sdpa, "speedup": ms_sdpa / ms, "tflops": fl / (ms * 1e-3) / 1e12,
                       "tflops_kernel_only": fl / (ms_k * 1e-3) / 1e12, "mem_mb": peak_mb(ours),
                       "mem_mb_sdpa": peak_mb(lambda: sdpa_dual(q, k, v, qt, kt, vt, mask, causal))}
                rows.append(row)
                print(f"L={L:5d} mask={kind:9s} causal={str(causal):5s} {'ok ' if ok else 'FAIL'} "
                      f"primal {acc['primal']:.2e} tangent {acc['tangent']:.2e} grads {max(acc['dq'], acc['dk'], acc['dv']):.2e} | "
                      f"{ms:7.3f} ms ({ms_k:7.3f} kernel only) sdpa {ms_sdpa:8.3f} ms x{ms_sdpa / ms:5.1f} | "
                      f"{row['tflops']:6.1f} TFLOP/s | {row['mem_mb']:7.1f} MB vs {row['mem_mb_sdpa']:8.1f} MB", flush=True)
    n_ok = sum(r["ok"] for r in rows)
    stats = summary_statistics(rows)
    print(summary_table(rows))
    print(mask_comparison_table(rows))
    print(f"\naccuracy: {n_ok}/{len(rows)} passed; speed-up over math SDPA: mean {stats['speedup_mean']:.2f}x, "
          f"min {stats['speedup_min']:.2f}x, max {stats['speedup_max']:.2f}x")
    if args.json:
        with open(args.json, "w") as f:
            json.dump({"dtype": args.dtype, "bsz": B, "heads": H, "head_dim": D, "tolerance": TOLERANCE[args.dtype],
                       "passed": n_ok, "cases": len(rows), **stats, "rows": rows}, f, indent=1)
    return rows


def summary_table(rows) -> str:
    """The reference's summary table (its test file, lines 883-937): one line per case and method."""
    out = ["", "=" * 110, "BENCHMARK SUMMARY", "=" * 110,
           f"{'Seq Len':<10} {'Causal':<8} {'Mask':<10} {'Method':<10} {'Time (ms)':<12} {'Mem (MB)':<12} {'TFLOP/s':<12} "
           f"{'Max Error':<12} {'Grad Check':<10}", "-" * 110]
    for r in sorted(rows, key=lambda r: (r["L"], r["causal"], r["mask"])):
        fl = r["tflops"] * r["ms"]  # TFLOP/s x ms: the case's FLOP count in units of 1e9
        out.append(f"{r['L']:<10} {str(r['causal']):<8} {r['mask']:<10} {'sdpa':<10} {r['ms_sdpa_math']:<12.3f} "
                   f"{r['mem_mb_sdpa']:<12.2f} {fl / r['ms_sdpa_math']:<12.2f} {'baseline':<12} {'N/A':<10}")
        worst = max(r["primal"], r["tangent"])
        out.append(f"{r['L']:<10} {str(r['causal']):<8} {r['mask']:<10} {'jvp_attn':<10} {r['ms']:<12.3f} "
                   f"{r['mem_mb']:<12.2f} {r['tflops']:<12.2f} {worst:<12.2e} {'ok' if r['ok'] else 'FAIL':<10}")
        out.append("")
    return "\n".join(out)


def mask_comparison_table(rows) -> str:
    """The reference's mask-type table (lines 940-976): time by mask type, relative to no mask."""
    out = ["", "=" * 80, "MASK TYPE PERFORMANCE COMPARISON", "=" * 80,
           f"{'Seq Len':<10} {'Causal':<8} {'Method':<10} {'No Mask':<15} {'Boolean Mask':<15} {'Additive Mask':<15}", "-" * 80]
    by = {}
    for r in rows:
        by.setdefault((r["L"], r["causal"]), {})[r["mask"]] = r["ms"]
    for (L, causal), t in sorted(by.items()):
        cell = lambda k: "N/A" if k not in t else (f"{t[k]:.2f} ms" + (f" ({t[k] / t['none']:.2f}x)" if k != "none" and "none" in t else ""))  # noqa: E731
        out.append(f"{L:<10} {str(causal):<8} {'jvp_attn':<10} {cell('none'):<15} {cell('boolean'):<15} {cell('additive'):<15}")
    return "\n".join(out)


def summary_statistics(rows) -> dict:
    """Speed-up over math SDPA (mean / min / max) and the worst errors, as the reference's closing statistics."""
    sp = [r["speedup"] for r in rows] or [float("nan")]
    return {"speedup_mean": sum(sp) / len(sp), "speedup_min": min(sp), "speedup_max": max(sp),
            "max_primal_error": max((r["primal"] for r in rows), default=0.0),
            "max_tangent_error": max((r["tangent"] for r in rows), default=0.0),
            "max_grad_error": max((max(r["dq"], r["dk"], r["dv"]) for r in rows), default=0.0)}


def plot_report(rows, dtype: str, out_dir: str, masks: bool = True):
    """The reference's two figures (its test file, lines 977-1091) from the rows of ``run``: for every
    (causal, mask) configuration one panel with the speed-up over math SDPA per sequence length, and one with the
    peak memory of one call of either method.  Returns the two file names (named as the reference names them)."""
    import os

    import matplotlib

    matplotlib.use("Agg")  # files only: no display on a GPU box
    import matplotlib.pyplot as plt

    panels = {}
    for r in rows:
        panels.setdefault((r["causal"], r["mask"]), []).append(r)
    os.makedirs(out_dir, exist_ok=True)
    suffix = "_with_masks" if masks else ""
    paths = [os.path.join(out_dir, f"{dtype}_jvp_attention_{what}{suffix}.png") for what in ("perf", "mem")]
    n = max(len(panels), 1)
    fig_p, ax_p = plt.subplots(1, n, figsize=(6 * n, 5), squeeze=False)
    fig_m, ax_m = plt.subplots(1, n, figsize=(6 * n, 5), squeeze=False)
    fig_p.suptitle("Speed-up of the fused dual forward over math SDPA under forward-mode AD")
    fig_m.suptitle("Peak memory of one call")
    for col, ((causal, mask), rs) in enumerate(sorted(panels.items(), key=lambda kv: (kv[0][0], kv[0][1]))):
        rs = sorted(rs, key=lambda r: r["L"])
        xs = list(range(len(rs)))
        labels = [str(r["L"]) for r in rs]
        title = f"causal={causal}, mask={mask}"
        a = ax_p[0, col]
        bars = a.bar(xs, [r["speedup"] for r in rs], width=0.5, color="tab:green")
        a.bar_label(bars, labels=[f"{r['speedup']:.1f}x" for r in rs])
        a.axhline(1.0, color="grey", linestyle="--")
        a.set(title=title, xlabel="sequence length", ylabel="math SDPA time / JVP attention time", xticks=xs, xticklabels=labels)
        b = ax_m[0, col]
        w = 0.38
        b1 = b.bar([x - w / 2 for x in xs], [r["mem_mb_sdpa"] for r in rs], w, label="math SDPA")
        b2 = b.bar([x + w / 2 for x in xs], [r["mem_mb"] for r in rs], w, label="JVP attention")
        b.bar_label(b1, fmt="%.0f", padding=2)
        b.bar_label(b2, fmt="%.0f", padding=2)
        b.set(title=title, xlabel="sequence length", ylabel="peak allocated memory (MB)", xticks=xs, xticklabels=labels)
        b.set_yscale("log")
        b.legend()
    for fig, path in ((fig_p, paths[0]), (fig_m, paths[1])):
        fig.tight_layout(rect=[0, 0.02, 1, 0.95])
        fig.savefig(path, dpi=120)
        plt.close(fig)
    return paths


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--dtype", default="bfloat16", choices=list(DTYPES))
    ap.add_argument("--bsz", type=int, default=2)
    ap.add_argument("--model-dim", type=int, default=768)
    ap.add_argument("--head-dim", type=int, default=64)
    ap.add_argument("--seq-lengths", type=int, nargs="+", default=[32, 64, 128, 256, 512, 1024, 2048])
    ap.add_argument("--no-masks", action="store_true")
    ap.add_argument("--no-timing", action="store_true", help="one call per case instead of 10 + 100: accuracy only")
    ap.add_argument("--json", default=None)
    ap.add_argument("--plots", default=None, metavar="DIR", help="draw the speed-up and memory figures into DIR (needs matplotlib)")
    args = ap.parse_args()
    rows = run(args)
    if args.plots:
        for path in plot_report(rows, args.dtype, args.plots, not args.no_masks):
            print("wrote", path)


if __name__ == "__main__":
    main()
