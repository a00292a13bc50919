#!/usr/bin/env python3
"""Headline benchmark: fused gated-MLP forward+backward on one MI355X.

Workload (the configuration the baseline metric is quoted on): fp16, M=8192 tokens, K=4096,
N=14336 (Llama-3-8B MLP), bias=False, dropout_p=0; one step = `y = mlp(x); y.backward(dY)` with a
dense upstream gradient.  FLOP model: 18*M*N*K per step (3 forward + 6 backward GEMMs), the same
count as the reference's `9 * 2 * M * N * K` (src/triton_gated_mlp/benchmark.py:86).

Prints ONE JSON line.  `roofline` covers the dominant kernel (the grouped launch of the three
weight-gradient GEMMs, a third of the step: 6*M*N*K FLOP per launch) timed with events on the launch
stream; `kernels` lists every launch of a step the same way; `cpu_baseline` times the CPU oracle on
a bounded sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "triton-gated-mlp_amd"))
sys.path.insert(0, str(ROOT))

import torch  # noqa: E402

PEAK_MFMA_F16_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA
PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E

M, K, N = 8192, 4096, 14336
DTYPE = torch.float16
# rocprofv3 --pmc FETCH_SIZE (x2.0, the factor a plain copy of known size reads) + WRITE_SIZE, per launch
# of the grouped weight-gradient kernel: 2 183 357 KiB x 2.0 + 344 064 KiB
DW_GROUP_TRAFFIC_BYTES = 4.824e9


def _median(v):
    v = sorted(v)
    return v[len(v) // 2]


def _event_time_ms(fn, reps, warmup=2):
    """Average duration of fn() in ms, measured with events on the stream fn launches on."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        start[i].record()
        fn()
        stop[i].record()
    torch.cuda.synchronize()
    t = [a.elapsed_time(b) for a, b in zip(start, stop)]
    return sum(t) / len(t), _median(t)


def _make_module(dev):
    from triton_gated_mlp import FusedGatedMLP

    g = torch.Generator().manual_seed(0)
    mlp = FusedGatedMLP(hidden_size=K, intermediate_size=N, bias=False, dropout_p=0.0)
    with torch.no_grad():
        mlp.gate_proj.weight.copy_(0.02 * torch.randn(N, K, generator=g))
        mlp.up_proj.weight.copy_(0.02 * torch.randn(N, K, generator=g))
        mlp.down_proj.weight.copy_(0.02 * torch.randn(K, N, generator=g))
    mlp = mlp.to(dev).to(DTYPE)
    x = torch.randn(M, K, generator=g).to(DTYPE).to(dev).requires_grad_(True)
    dY = torch.randn(M, K, generator=g).to(DTYPE).to(dev)
    return mlp, x, dY


def _kernel_breakdown(mlp, x, dY, reps):
    """Per-launch timings of one step through the operator layer (same kernels the module runs)."""
    from triton_gated_mlp.ops import bwd as B
    from triton_gated_mlp.ops import fwd as F

    Wg, Wu, Wd = mlp.gate_proj.weight.detach(), mlp.up_proj.weight.detach(), mlp.down_proj.weight.detach()
    xd = x.detach()
    hs = F.gateup_fwd(xd, Wg, None, Wu, None, save_activations=True)
    dg, du = B.dh_bwd(dY, Wd, hs.gate, hs.up)
    mnk2 = 2.0 * M * N * K
    launches = [
        ("gateup_fwd", lambda: F.gateup_fwd(xd, Wg, None, Wu, None, save_activations=True), 2 * mnk2),
        ("down_fwd", lambda: F.linear_fwd(hs.hidden, Wd), mnk2),
        ("dh_bwd", lambda: B.dh_bwd(dY, Wd, hs.gate, hs.up), mnk2),
        ("dx_bwd", lambda: B.dx_bwd(dg, du, Wg, Wu), 2 * mnk2),
        ("dw_gate_up_down_grouped", lambda: B.dw_bwd_grouped([(dg, xd), (du, xd), (dY, hs.hidden)]), 3 * mnk2),
    ]
    out = {}
    for name, fn, flop in launches:
        avg, med = _event_time_ms(fn, reps)
        out[name] = {"ms": round(avg, 4), "tflops": round(flop / avg / 1e9, 1), "frac_mfma_peak": round(flop / avg / 1e9 / PEAK_MFMA_F16_TFLOPS, 4)}
    return out


def _decode_line(dev, reps=20):
    """Skinny-M forward (M=16, K=8192, N=28672, fp16): achieved HBM GB/s on algorithmic bytes."""
    from triton_gated_mlp.ops import fwd as F

    m, k, n = 16, 8192, 28672
    g = torch.Generator().manual_seed(1)
    x = torch.randn(m, k, generator=g).half().to(dev)
    Wg = torch.empty(n, k, dtype=torch.float16, device=dev).normal_(0, 0.02)
    Wu = torch.empty(n, k, dtype=torch.float16, device=dev).normal_(0, 0.02)
    Wd = torch.empty(k, n, dtype=torch.float16, device=dev).normal_(0, 0.02)
    nbytes = 3 * k * n * 2 + m * k * 2 + 2 * m * n * 2 + m * k * 2
    avg, med = _event_time_ms(lambda: F.decode_fwd(x, Wg, None, Wu, None, Wd, None), reps, warmup=3)
    return {"workload": "fp16 decode fwd M=16 K=8192 N=28672", "us": round(avg * 1e3, 1), "bytes": nbytes,
            "gbps": round(nbytes / avg / 1e6, 1), "frac_hbm_peak": round(nbytes / avg / 1e6 / PEAK_HBM_GBPS, 4)}


def _other_configs(dev):
    """The remaining baseline configurations, timed with events (median of 10 after 3 warm-ups)."""
    from triton_gated_mlp import FusedGatedMLP

    out = {}
    for name, (m, k, n, dt, bias, p, bwd) in {
        "cfg2_fp16_fwd_M4096_K4096_N11008": (4096, 4096, 11008, torch.float16, False, 0.0, False),
        "cfg4_bf16_fwdbwd_bias_dropout_M2048_K2048_N5632": (2048, 2048, 5632, torch.bfloat16, True, 0.1, True),
    }.items():
        mlp = FusedGatedMLP(hidden_size=k, intermediate_size=n, bias=bias, dropout_p=p).to(dev).to(dt)
        mlp.train(bwd)
        mlp.dropout_seed = 1234
        x = torch.randn(m, k, device=dev, dtype=dt, requires_grad=bwd)
        dy = torch.randn(m, k, device=dev, dtype=dt)
        params = list(mlp.parameters())

        def step():
            if bwd:
                x.grad = None
                for q in params:
                    q.grad = None
                mlp(x).backward(dy)
            else:
                with torch.no_grad():
                    mlp(x)

        avg, med = _event_time_ms(step, 10, warmup=3)
        flop = (18.0 if bwd else 6.0) * m * n * k
        out[name] = {"ms": round(med, 4), "tflops": round(flop / med / 1e9, 1),
                     "frac_mfma_peak": round(flop / med / 1e9 / PEAK_MFMA_F16_TFLOPS, 4)}
        del mlp, x, dy, params
    out.update(_edge_shapes(dev))
    return out


def _edge_shapes(dev):
    """Shapes off the tile grid, next to torch's own operators (rocBLAS/hipBLASLt) on the same GPU:
    a ragged token count at the headline widths (fwd+bwd), a short batch at the decode widths
    (forward; the down projection splits its reduction) and a batch whose 2.3 GB activations are
    beyond 32-bit byte offsets (fwd+bwd; the module runs it as two row chunks)."""
    from triton_gated_mlp import EagerGatedMLP, FusedGatedMLP

    out = {}
    for name, (m, k, n, bwd) in {
        "ragged_fp16_fwdbwd_M8191_K4096_N14336": (8191, 4096, 14336, True),
        "short_batch_fp16_fwd_M32_K8192_N28672": (32, 8192, 28672, False),
        "tall_batch_fp16_fwdbwd_M40960_K8192_N28672": (40960, 8192, 28672, True),
    }.items():
        fused = FusedGatedMLP(hidden_size=k, intermediate_size=n, bias=False).to(dev).to(DTYPE)
        eager = EagerGatedMLP(hidden_size=k, intermediate_size=n, bias=False).to(dev).to(DTYPE)
        x = torch.randn(m, k, device=dev, dtype=DTYPE, requires_grad=bwd)
        dy = torch.randn(m, k, device=dev, dtype=DTYPE)
        res = {}
        for label, mod in (("ms", fused), ("torch_eager_ms", eager)):
            params = list(mod.parameters())

            def step():
                if bwd:
                    x.grad = None
                    for q in params:
                        q.grad = None
                    mod(x).backward(dy)
                else:
                    with torch.no_grad():
                        mod(x)

            reps = 10 if m <= 8192 else 3
            res[label] = round(_event_time_ms(step, reps, warmup=min(3, reps))[1], 4)
        flop = (18.0 if bwd else 6.0) * m * n * k
        res["tflops"] = round(flop / res["ms"] / 1e9, 1)
        out[name] = res
        del fused, eager, x, dy
    return out


def _cpu_baseline():
    """CPU oracle (fp32 restatement of the eager module, closed-form backward) on a bounded sample:
    the first 1024 of the 8192 token rows, same K and N, forward+backward."""
    from oracle import eager as oracle

    ms = 1024
    g = torch.Generator().manual_seed(0)
    Wg = 0.02 * torch.randn(N, K, generator=g)
    Wu = 0.02 * torch.randn(N, K, generator=g)
    Wd = 0.02 * torch.randn(K, N, generator=g)
    x = torch.randn(ms, K, generator=g)
    dY = torch.randn(ms, K, generator=g)
    times = []
    for i in range(3):
        t0 = time.perf_counter()
        oracle.backward(x, Wg, None, Wu, None, Wd, None, dY)
        times.append(time.perf_counter() - t0)
    t = _median(times[1:]) if len(times) > 1 else times[0]
    flop = 18.0 * ms * N * K
    model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": round(flop / t / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"fwd+bwd of rows 0..{ms - 1} of the workload (M={ms}, K={K}, N={N}), fp32 torch-CPU oracle, "
                      f"median of 2 after 1 warm-up, {t * 1e3:.0f} ms/step",
            "os_cpu_count": os.cpu_count(), "cpu_model": model}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip per-kernel breakdown and decode line")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (reference point for FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an AMD GPU (no CPU fallback for the fused path)")
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)

    if args.calibration_copy:
        src = torch.ones(256 * 1024 * 1024, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    mlp, x, dY = _make_module(dev)
    params = list(mlp.parameters())

    def step():
        x.grad = None
        for p in params:
            p.grad = None
        y = mlp(x)
        y.backward(dY)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    flop_step = 18.0 * M * N * K
    tflops = flop_step / (ms_per_step * 1e-3) / 1e12

    # dominant kernel: dW_gate, dW_up and dW_down as one grouped launch (6*M*N*K FLOP), events on
    # the launch stream
    from triton_gated_mlp.ops import bwd as B
    from triton_gated_mlp.ops import fwd as F

    Wg, Wu, Wd = mlp.gate_proj.weight.detach(), mlp.up_proj.weight.detach(), mlp.down_proj.weight.detach()
    xd = x.detach()
    hs = F.gateup_fwd(xd, Wg, None, Wu, None, save_activations=True)
    dg, du = B.dh_bwd(dY, Wd, hs.gate, hs.up)
    avg, med = _event_time_ms(lambda: B.dw_bwd_grouped([(dg, xd), (du, xd), (dY, hs.hidden)]), max(args.steps, 10))
    del dg, du, hs
    dom_flop = 6.0 * M * N * K
    roofline = {"kernel": "gemm_group_kernel_pipelined<f16,256,256,16,...,EpiStore> (dW_gate + dW_up + dW_down, one grouped launch)",
                "bound": "mfma", "achieved": round(dom_flop / avg / 1e9, 1), "peak": PEAK_MFMA_F16_TFLOPS,
                "unit": "TFLOP/s", "frac": round(dom_flop / avg / 1e9 / PEAK_MFMA_F16_TFLOPS, 4),
                "avg_launch_ms": round(avg, 4), "flop_per_launch": dom_flop, "traffic": DW_GROUP_TRAFFIC_BYTES,
                "traffic_note": "HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                "(profiles/gemm_hbm_traffic_fp16_M8192_K4096_N14336.txt); algorithmic bytes are 1.258e9"}

    line = {
        "metric": "fwd+bwd TFLOP/s & % MFMA peak, fp16 M=8192 K=4096 N=14336 (1 GPU)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "frac_mfma_peak": round(tflops / PEAK_MFMA_F16_TFLOPS, 4),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "fp16 fwd+bwd gated MLP, M=8192 K=4096 N=14336, bias=False, dropout_p=0 (Llama-3-8B MLP)",
                   "M": M, "K": K, "N": N, "flop_per_step": flop_step},
        "roofline": roofline,
    }
    if not args.no_extras:
        line["kernels"] = _kernel_breakdown(mlp, x, dY, 10)
        line["decode"] = _decode_line(dev)
        line["other_configs"] = _other_configs(dev)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = _cpu_baseline()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
