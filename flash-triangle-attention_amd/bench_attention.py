"""Sequence-length sweep with the shape of upstream's bench_attention (flash_tt_attn.py:714-843):
batch 4, 8 heads, head dim 32, fp16, N(0,1) inputs, sm_scale = 1.3; providers "hip" (this library;
the upstream names "triton" and "triton-fp16" are accepted for it) and "vanilla-torch" (the naive
O(L^3) formulation, reference_tt_attn); modes "fwd" and "bwd" (the backward alone, of an output
computed before the timed region, as upstream :787-790); metrics "time" (ms) and "memory" (peak GB
allocated while the provider ran, inputs included, as upstream :724-731).

    python bench_attention.py                      # tables on stdout
    python bench_attention.py --out results_dir    # also one CSV and one PNG per (mode, metric), named as
                                                   # upstream's test_results/, and a results.html over them

Sequence lengths must be multiples of 128 for the library (upstream's points below 128 ran kernels
without masking on an empty backward grid); out of memory gives inf (memory) or nan (time), as
upstream :836-841.  Timing: median of HIP-event timings after warm-up, caches not flushed.
"""
from __future__ import annotations

import argparse
import os
import statistics
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from flash_tt_attn import attention, reference_tt_attn  # noqa: E402

HIP_PROVIDERS = ("hip", "triton", "triton-fp16")
LINE_NAMES = {"hip": "HIP [FP16]", "vanilla-torch": "Vanilla PyTorch"}


def do_bench(fn, warmup: int = 5, rep: int = 20) -> float:
    """Median run time of fn() in ms (HIP events on the current stream)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(rep):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    return statistics.median(times)


# Element type and softmax scale of the sweep: upstream's values (:764, :783); the command line can
# change them (--dtype bf16, --sm-scale), and switch on what upstream does not have (--dropout P: dropout
# on the attention weights with a fixed seed; --precise: the precise fp16 backward).
DTYPE = torch.float16
SM_SCALE = 1.3
DROPOUT_P = 0.0


def bench_attention(B, H, L, D, mode, provider, device=None, metric="time"):
    """One point of the sweep; same arguments and return conventions as upstream :762."""
    assert mode in ["fwd", "bwd"]
    device = torch.device("cuda") if device is None else torch.device(device)
    dtype = DTYPE
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    try:
        q = torch.randn((B, H, L, L, D), dtype=dtype, device=device, requires_grad=True)
        k = torch.randn((B, H, L, L, D), dtype=dtype, device=device, requires_grad=True)
        v = torch.randn((B, H, L, L, D), dtype=dtype, device=device, requires_grad=True)
        b = torch.randn((B, H, L, L), dtype=dtype, device=device, requires_grad=True)
        sm_scale = SM_SCALE
        if provider in HIP_PROVIDERS:
            fn = (lambda: attention(q, k, v, b, sm_scale, DROPOUT_P, 7)) if DROPOUT_P > 0.0 else (lambda: attention(q, k, v, b, sm_scale))
        elif provider == "vanilla-torch":
            fn = lambda: reference_tt_attn(q, k, v, b, sm_scale)
        else:
            raise ValueError(f"Invalid provider: {provider}")
        if mode == "bwd":
            o = fn()
            do = torch.randn_like(o)

            def fn():
                q.grad = k.grad = v.grad = b.grad = None  # time the backward, not the += into .grad
                o.backward(do, retain_graph=True)
        ms = do_bench(fn)
        torch.cuda.synchronize()
        peak_gb = torch.cuda.max_memory_allocated() / 2**30
    except torch.cuda.OutOfMemoryError:
        return float("inf") if metric == "memory" else float("nan")
    if metric == "memory":
        return peak_gb
    if metric == "time":
        return ms
    raise NotImplementedError("metrics: 'time' (ms) and 'memory' (GB)")


def _plot(path, title, rows, providers, ylabel):
    """One line per provider over L, log-log like upstream's perf_report configuration (:733-760).  Returns
    False where matplotlib is missing (the CSV tables are then all that is written)."""
    try:
        import matplotlib
        matplotlib.use("Agg")
        import matplotlib.pyplot as plt
    except ImportError:
        return False
    fig, ax = plt.subplots(figsize=(6, 4))
    for prov, style in zip(providers, ("-", "--", ":", "-.")):
        pts = [(L, vals[prov]) for L, vals in rows if vals[prov] == vals[prov] and vals[prov] != float("inf")]
        if pts:
            ax.plot([x for x, _ in pts], [y for _, y in pts], style, marker="o", label=LINE_NAMES[prov])
    ax.set_xscale("log", base=2)
    ax.set_yscale("log")
    ax.set_xlabel("L")
    ax.set_ylabel(ylabel)
    ax.set_title(title)
    ax.legend()
    fig.tight_layout()
    fig.savefig(path, dpi=100)
    plt.close(fig)
    return True


def sweep(B=4, H=8, D=32, Ls=(128, 256, 512, 1024), providers=("hip", "vanilla-torch"), vanilla_max_L=512, out=None):
    """Runs every (mode, metric, L, provider) point; returns {(mode, metric): [(L, {provider: value})]}."""
    tables = {}
    images = []
    for mode in ("fwd", "bwd"):
        for metric in ("memory", "time"):
            rows = []
            for L in Ls:
                vals = {}
                for prov in providers:
                    if prov == "vanilla-torch" and L > vanilla_max_L:
                        vals[prov] = float("nan")  # O(L^3) memory: not attempted
                    else:
                        vals[prov] = bench_attention(B, H, L, D, mode, prov, metric=metric)
                rows.append((L, vals))
                print(f"{mode:3s} {metric:6s} L={L:5d} " + " ".join(f"{LINE_NAMES[p]}={vals[p]:.6f}" for p in providers), flush=True)
            tables[(mode, metric)] = rows
            if out:
                os.makedirs(out, exist_ok=True)
                name = f"fused-attention-batch{B}-head{H}-d{D}-{mode}-{'latency' if metric == 'time' else 'memory'}.csv"
                with open(os.path.join(out, name), "w") as f:
                    f.write("L," + ",".join(LINE_NAMES[p] for p in providers) + "\n")
                    for L, vals in rows:
                        f.write(f"{float(L):.6f}," + ",".join(f"{vals[p]:.6f}" for p in providers) + "\n")
                png = name[:-4] + ".png"
                if _plot(os.path.join(out, png), name[:-4], rows, providers, "ms" if metric == "time" else "GB"):
                    images.append(png)
    if out and images:
        with open(os.path.join(out, "results.html"), "w") as f:
            f.write("<html><body>\n" + "".join(f'<image src="{png}"/>\n' for png in images) + "</body></html>\n")
    return tables


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--B", type=int, default=4)
    ap.add_argument("--H", type=int, default=8)
    ap.add_argument("--D", type=int, default=32)
    ap.add_argument("--L", type=int, nargs="*", default=[128, 256, 512, 1024])
    ap.add_argument("--vanilla-max-L", type=int, default=512, help="largest L the naive provider is run at")
    ap.add_argument("--out", default=None, help="directory for the CSV tables")
    ap.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16")
    ap.add_argument("--sm-scale", type=float, default=SM_SCALE)
    ap.add_argument("--dropout", type=float, default=0.0, help="dropout probability on the attention weights (library only)")
    ap.add_argument("--precise", action="store_true", help="the precise fp16 backward (library only)")
    a = ap.parse_args()
    DTYPE = torch.bfloat16 if a.dtype == "bf16" else torch.float16
    LINE_NAMES["hip"] = f"HIP [{a.dtype.upper()}]"
    SM_SCALE = a.sm_scale
    DROPOUT_P = a.dropout
    if a.precise:
        import flash_tt_attn
        flash_tt_attn.PRECISE_BACKWARD = True
    if not torch.cuda.is_available():
        sys.exit("bench_attention.py needs a GPU (there is no CPU path for the library)")
    sweep(a.B, a.H, a.D, tuple(a.L), vanilla_max_L=a.vanilla_max_L, out=a.out)
