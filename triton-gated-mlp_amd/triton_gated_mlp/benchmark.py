"""Throughput and peak-memory sweep: EagerGatedMLP (torch, vendor BLAS) vs FusedGatedMLP on one GPU.

Same experiment as the reference's script (src/triton_gated_mlp/benchmark.py:27-123): fp16,
bias=False, dropout_p=0, cubes M = N = K in {32, 64, ..., 4096}, one step = forward +
`out.sum().backward()`, TFLOPS = 9 * 2 * M * N * K / t, and peak allocated memory of one step (above
what was allocated before it; the absolute peak the reference prints is kept as `<provider>_total`).
Timing follows the same recipe as triton.testing.do_bench (warm-up, a cache flush between
repetitions, median and 20 % / 80 % quantiles) without importing triton.

    python -m triton_gated_mlp.benchmark [--out DIR] [--max-exp 12] [--plots]

Prints both tables and writes benchmark_tflops.csv / benchmark_memory.csv (and PNG bar charts with
--plots when matplotlib is importable).
"""

from __future__ import annotations

import argparse
import csv
from pathlib import Path

import torch

from .gated_mlp import EagerGatedMLP, FusedGatedMLP
from .utils import get_device

PROVIDERS = {"torch": EagerGatedMLP, "fused": FusedGatedMLP}
DTYPE = torch.float16


def do_bench(fn, warmup_ms: float = 25.0, rep_ms: float = 100.0, quantiles=(0.5, 0.2, 0.8)):
    """Median / quantile run time of fn() in ms; a 512 MB write evicts L2 and the 256 MB
    Infinity Cache between repetitions."""
    flush = torch.empty(512 * 1024 * 1024, dtype=torch.int8, device="cuda")
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(5):
        flush.zero_()
        fn()
    b.record()
    torch.cuda.synchronize()
    est = max(a.elapsed_time(b) / 5, 1e-3)
    n_warm = max(1, int(warmup_ms / est))
    n_rep = max(5, min(200, int(rep_ms / est)))
    for _ in range(n_warm):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    for i in range(n_rep):
        flush.zero_()
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    t = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, stops)], dtype=torch.float64)
    return [torch.quantile(t, q).item() for q in quantiles]


def make_mlp(provider: str, N: int, K: int, device):
    return PROVIDERS[provider](hidden_size=K, intermediate_size=N, dropout_p=0.0, bias=False).to(device).to(DTYPE)


def step(mlp, x):
    x.grad = None
    for p in mlp.parameters():
        p.grad = None
    mlp(x).sum().backward()


def sweep(sizes, device):
    perf, mem = [], []
    for s in sizes:
        M = N = K = s
        row_p, row_m = {"N": s}, {"N": s}
        for provider in PROVIDERS:
            mlp = make_mlp(provider, N, K, device)
            x = torch.randn((M, K), device=device, dtype=DTYPE, requires_grad=True)
            ms, lo, hi = do_bench(lambda: step(mlp, x))
            tf = lambda t: 9 * 2 * M * N * K * 1e-12 / (t * 1e-3)
            row_p[provider], row_p[provider + "_min"], row_p[provider + "_max"] = tf(ms), tf(hi), tf(lo)
            x.grad = None
            for p in mlp.parameters():
                p.grad = None
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            torch.cuda.reset_peak_memory_stats(device)
            # What is allocated before the step (parameters, x, and whatever the process holds for
            # good, such as the vendor BLAS workspace torch keeps once the eager module has run) is
            # not the module's doing: the column is the step's own peak; the absolute peak, which
            # is what the reference's script prints, goes to <provider>_total.
            before = torch.cuda.memory_allocated(device)
            step(mlp, x)
            torch.cuda.synchronize()
            peak = torch.cuda.max_memory_allocated(device)
            row_m[provider] = (peak - before) / 1024 / 1024
            row_m[provider + "_total"] = peak / 1024 / 1024
            del mlp, x
        print(f"M=N=K={s:5d}  " + "  ".join(f"{p}: {row_p[p]:8.2f} TFLOPS {row_m[p]:9.1f} MB" for p in PROVIDERS), flush=True)
        perf.append(row_p)
        mem.append(row_m)
    return perf, mem


def _write_csv(path: Path, rows):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0]))
        w.writeheader()
        w.writerows(rows)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--out", default=".", help="directory for the CSV (and PNG) files")
    ap.add_argument("--min-exp", type=int, default=5)
    ap.add_argument("--max-exp", type=int, default=12)
    ap.add_argument("--plots", action="store_true")
    args = ap.parse_args(argv)
    device = get_device()
    if device.type != "cuda":
        raise SystemExit("the benchmark needs a GPU: FusedGatedMLP has no CPU implementation")
    sizes = [2**i for i in range(args.min_exp, args.max_exp + 1)]
    perf, mem = sweep(sizes, device)
    out = Path(args.out)
    out.mkdir(parents=True, exist_ok=True)
    _write_csv(out / "benchmark_tflops.csv", perf)
    _write_csv(out / "benchmark_memory.csv", mem)
    if args.plots:
        try:
            import matplotlib

            matplotlib.use("Agg")
            import matplotlib.pyplot as plt
        except ImportError:
            print("matplotlib is not importable: skipping the plots")
            return
        for rows, ylabel, name in ((perf, "TFLOPS", "benchmark_tflops.png"), (mem, "peak memory (MB)", "benchmark_memory.png")):
            fig, ax = plt.subplots()
            w = 0.4
            for i, p in enumerate(PROVIDERS):
                ax.bar([j + (i - 0.5) * w for j in range(len(rows))], [r[p] for r in rows], w, label=p)
            ax.set_xticks(range(len(rows)), [str(r["N"]) for r in rows])
            ax.set_xlabel("M = N = K")
            ax.set_ylabel(ylabel)
            ax.legend()
            fig.tight_layout()
            fig.savefig(out / name)


if __name__ == "__main__":
    main()
