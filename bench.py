#!/usr/bin/env python3
"""Headline benchmark: fused gated-MLP forward+backward on one MI355X.

Workload (the configuration the baseline metric is quoted on): fp16, M=8192 tokens, K=4096,
N=14336 (Llama-3-8B MLP), bias=False, dropout_p=0; one step = `y = mlp(x); y.backward(dY)` with a
dense upstream gradient.  FLOP model: 18*M*N*K per step (3 forward + 6 backward GEMMs), the same
count as the reference's `9 * 2 * M * N * K` (src/triton_gated_mlp/benchmark.py:86).

Prints ONE JSON line.
  value / ms_per_step   wall clock over exactly --steps steps between two synchronisations (no cache
                        flush inside the timed region: the step's working set, 1.5 GB, is six times
                        the 256 MB memory-side cache)
  step_quantiles        the same step timed one at a time with events, a 512 MB write between
                        repetitions (the recipe of triton.testing.do_bench that the reference's
                        script uses, src/triton_gated_mlp/benchmark.py:82-85): median, p20, p80
  roofline              the launch that takes the largest share of a step: dW_gate, dW_up and dW_down
                        through gmlp_dw_bwd_grouped (6*M*N*K FLOP), events on the launch stream
  kernels               every launch of a step the same way
  configs               the other baseline configurations, each with quantiles, its own roofline
                        block and the CPU oracle timed beside it on a stated sample
  cpu_baseline          the CPU oracle on a bounded sample of the headline workload
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
PEAK_MFMA_F32_TFLOPS = 157.3  # MI355X dense fp32 MFMA
PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E

M, K, N = 8192, 4096, 14336
DTYPE = torch.float16
DW_GROUP_ALGORITHMIC_BYTES = 1.258e9  # dG, dU, dY, H once, x twice, three dW once
# HBM-side bytes per call (`roofline.traffic`) are not measured by this script: they come from two
# `rocprofv3 --pmc` runs of it (FETCH_SIZE, WRITE_SIZE), summarised in the files below, each of
# which carries one line `traffic_bytes_per_call = <bytes>`.  The JSON line names the file and its
# git blob hash next to the figure, so a figure that predates a kernel change shows.
DW_GROUP_TRAFFIC_PROFILE = "profiles/gemm_hbm_traffic_fp16_M8192_K4096_N14336.txt"
DECODE_TRAFFIC_PROFILE = "profiles/decode_hbm_traffic_fp16_M16_K8192_N28672.txt"


def _traffic_from_profile(rel):
    """(bytes per call or None, provenance) from a committed rocprofv3 summary."""
    import hashlib
    import re

    path = ROOT / rel
    try:
        raw = path.read_bytes()
    except OSError:
        return None, {"file": rel, "error": "missing"}
    m = re.search(rb"^traffic_bytes_per_call\s*=\s*([0-9.eE+]+)", raw, flags=re.M)
    blob = hashlib.sha1(b"blob %d\0" % len(raw) + raw).hexdigest()
    note = "HBM-side bytes per call from rocprofv3 --pmc FETCH_SIZE (x2.0) + WRITE_SIZE (x1.0), factors from a plain 256 MiB copy"
    return (float(m.group(1)) if m else None), {"file": rel, "git_blob": blob, "how": note}


_flush_buf = None


def _flush():
    """Evicts L2 and the 256 MB memory-side cache: a 512 MB write."""
    global _flush_buf
    if _flush_buf is None:
        _flush_buf = torch.empty(512 * 1024 * 1024, dtype=torch.int8, device="cuda")
    _flush_buf.zero_()


def _quantile(v, q):
    v = sorted(v)
    pos = q * (len(v) - 1)
    lo = int(pos)
    hi = min(lo + 1, len(v) - 1)
    return v[lo] + (v[hi] - v[lo]) * (pos - lo)


def _bench(fn, warmup_ms=25.0, rep_ms=100.0, min_reps=5, max_reps=200, flush=True):
    """Times fn() one call at a time with events on the current stream: enough warm-up calls for
    `warmup_ms`, enough repetitions for `rep_ms`, a cache flush before every repetition (outside the
    event pair).  Returns ms: p50, p20, p80, mean."""
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(3):
        fn()
    b.record()
    torch.cuda.synchronize()
    est = max(a.elapsed_time(b) / 3, 1e-3)
    for _ in range(max(1, min(1000, int(warmup_ms / est)))):
        fn()
    reps = max(min_reps, min(max_reps, int(rep_ms / est)))
    start = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        if flush:
            _flush()
        start[i].record()
        fn()
        stop[i].record()
    torch.cuda.synchronize()
    t = [s.elapsed_time(e) for s, e in zip(start, stop)]
    return {"p50": _quantile(t, 0.5), "p20": _quantile(t, 0.2), "p80": _quantile(t, 0.8), "mean": sum(t) / len(t),
            "reps": reps}


def _r(x, n=4):
    return round(x, n)


def _stated_inputs(mod, m, k, dev, dt, backward, seed=0):
    """Fills a gated-MLP module and makes its inputs from the distributions the baseline
    configurations state: weights ~ N(0, 0.02), biases ~ U(-0.01, 0.01), x ~ N(0, 1), upstream
    gradient ~ N(0, 1); seeded, generated on the device in fp32 and rounded to `dt`.  (Operand
    statistics matter to the timing: the chip runs these kernels at its power cap.)"""
    g = torch.Generator(device=dev).manual_seed(seed)
    with torch.no_grad():
        for lin in (mod.gate_proj, mod.up_proj, mod.down_proj):
            lin.weight.copy_(torch.empty(lin.weight.shape, device=dev).normal_(0.0, 0.02, generator=g))
            if lin.bias is not None:
                lin.bias.copy_(torch.empty(lin.bias.shape, device=dev).uniform_(-0.01, 0.01, generator=g))
    x = torch.empty(m, k, device=dev).normal_(0.0, 1.0, generator=g).to(dt).requires_grad_(backward)
    dy = torch.empty(m, k, device=dev).normal_(0.0, 1.0, generator=g).to(dt)
    return x, dy


def _make_module(dev):
    from triton_gated_mlp import FusedGatedMLP

    mlp = FusedGatedMLP(hidden_size=K, intermediate_size=N, bias=False, dropout_p=0.0).to(dev).to(DTYPE)
    x, dY = _stated_inputs(mlp, M, K, dev, DTYPE, True)
    return mlp, x, dY


def _mfma_block(flop, ms, peak=PEAK_MFMA_F16_TFLOPS):
    tf = flop / ms / 1e9
    return {"bound": "mfma", "achieved": _r(tf, 1), "peak": peak, "unit": "TFLOP/s", "frac": _r(tf / peak)}


def _kernel_breakdown(mlp, x, dY):
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
        t = _bench(fn, rep_ms=40.0, min_reps=10)
        out[name] = {"ms": _r(t["mean"]), "ms_p50": _r(t["p50"]), "tflops": _r(flop / t["mean"] / 1e9, 1),
                     "frac_mfma_peak": _r(flop / t["mean"] / 1e9 / PEAK_MFMA_F16_TFLOPS)}
    return out


def _cpu_info():
    model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"cores": torch.get_num_threads(), "os_cpu_count": os.cpu_count(), "cpu_model": model}


def _cpu_leg(m, k, n, backward, bias, p, flop_per_row, reps=2):
    """CPU oracle (fp32 restatement of the eager module, closed-form backward) on m rows of a
    configuration: 1 warm-up + `reps` timed, median."""
    from oracle import eager as oracle

    g = torch.Generator().manual_seed(0)
    Wg, Wu, Wd = 0.02 * torch.randn(n, k, generator=g), 0.02 * torch.randn(n, k, generator=g), 0.02 * torch.randn(k, n, generator=g)
    bg = bu = bd = None
    if bias:
        bg, bu, bd = [(torch.rand(c, generator=g) - 0.5) * 0.02 for c in (n, n, k)]
    x, dY = torch.randn(m, k, generator=g), torch.randn(m, k, generator=g)
    keep = (torch.rand(m, n, generator=g) >= p) if p > 0.0 else None
    times = []
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        if backward:
            oracle.backward(x, Wg, bg, Wu, bu, Wd, bd, dY, keep, p)
        else:
            oracle.forward(x, Wg, bg, Wu, bu, Wd, bd, keep, p)
        times.append(time.perf_counter() - t0)
    t = _quantile(times[1:], 0.5)
    return t, flop_per_row * m / t / 1e12


def _config_lines(dev):
    """The other baseline configurations.  GPU: quantiles with a cache flush between repetitions,
    inputs resident on the device.  CPU: the fp32 oracle on the stated row sample (same K, N)."""
    from oracle import eager as oracle
    from triton_gated_mlp import FusedGatedMLP
    from triton_gated_mlp.ops import fwd as F

    out = {}

    # cfg1: the reference's own CPU-runnable case (plumbing): fp32, forward only
    m, k, n = 128, 512, 256
    torch.manual_seed(0)
    ref = oracle.OracleGatedMLP(hidden_size=k, intermediate_size=n, bias=False, dropout_p=0.0).float()
    torch.manual_seed(0)
    x = torch.rand(m, k)
    with torch.no_grad():
        ref(x)
        t0 = time.perf_counter()
        for _ in range(20):
            y_ref = ref(x)
        cpu_ms = (time.perf_counter() - t0) / 20 * 1e3
    fused = FusedGatedMLP(hidden_size=k, intermediate_size=n, bias=False, dropout_p=0.0).float()
    fused.load_state_dict(ref.state_dict())
    fused = fused.to(dev)
    xd = x.to(dev)
    with torch.no_grad():
        y = fused(xd)
        t = _bench(lambda: fused(xd))
    flop = 6.0 * m * n * k
    out["cfg1_fp32_fwd_M128_K512_N256"] = {
        "gpu": {"ms_p50": _r(t["p50"], 5), "ms_p20": _r(t["p20"], 5), "ms_p80": _r(t["p80"], 5), "tflops": _r(flop / t["p50"] / 1e9, 3),
                "max_abs_err_vs_cpu": float((y.cpu() - y_ref).abs().max()),
                "roofline": dict(_mfma_block(flop, t["p50"], PEAK_MFMA_F32_TFLOPS), note="latency-bound: 1e8 FLOP, two launches")},
        "cpu": {"ms": _r(cpu_ms, 4), "tflops": _r(flop / cpu_ms / 1e9, 4), "sample": "the whole configuration, fp32 torch-CPU oracle, mean of 20"},
    }
    del fused, xd

    for name, (m, k, n, dt, bias, p, bwd, cpu_rows) in {
        "cfg2_fp16_fwd_M4096_K4096_N11008": (4096, 4096, 11008, torch.float16, False, 0.0, False, 1024),
        "cfg4_bf16_fwdbwd_bias_dropout_M2048_K2048_N5632": (2048, 2048, 5632, torch.bfloat16, True, 0.1, True, 1024),
    }.items():
        mlp = FusedGatedMLP(hidden_size=k, intermediate_size=n, bias=bias, dropout_p=p).to(dev).to(dt)
        mlp.train(bwd)
        mlp.dropout_seed = 1234
        x, dy = _stated_inputs(mlp, m, k, dev, dt, bwd)
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

        t = _bench(step)
        per_row = (18.0 if bwd else 6.0) * n * k
        flop = per_row * m
        cpu_t, cpu_tf = _cpu_leg(cpu_rows, k, n, bwd, bias, p, per_row)
        out[name] = {
            "gpu": {"ms_p50": _r(t["p50"]), "ms_p20": _r(t["p20"]), "ms_p80": _r(t["p80"]), "tflops": _r(flop / t["p50"] / 1e9, 1),
                    "cache_flush_between_reps": True, "roofline": _mfma_block(flop, t["p50"])},
            "cpu": {"ms": _r(cpu_t * 1e3, 1), "tflops": _r(cpu_tf, 4),
                    "sample": f"rows 0..{cpu_rows - 1} of {m} (same K, N), fp32 torch-CPU oracle, median of 2 after 1 warm-up"},
        }
        del mlp, x, dy, params

    # cfg5: skinny-M forward, memory-bound: every weight byte once
    m, k, n = 16, 8192, 28672
    g = torch.Generator().manual_seed(1)
    x = torch.randn(m, k, generator=g).half().to(dev)
    Wg = torch.empty(n, k, dtype=torch.float16, device=dev).normal_(0, 0.02)
    Wu = torch.empty(n, k, dtype=torch.float16, device=dev).normal_(0, 0.02)
    Wd = torch.empty(k, n, dtype=torch.float16, device=dev).normal_(0, 0.02)
    nbytes = 3 * k * n * 2 + m * k * 2 + 2 * m * n * 2 + m * k * 2
    traffic, traffic_src = _traffic_from_profile(DECODE_TRAFFIC_PROFILE)
    t = _bench(lambda: F.decode_fwd(x, Wg, None, Wu, None, Wd, None), rep_ms=30.0, min_reps=20)
    # CPU: one sixteenth of the intermediate width (the CPU is bound by reading the weights as well)
    cpu_n = n // 16
    cpu_t, cpu_tf = _cpu_leg(m, k, cpu_n, False, False, 0.0, 6.0 * cpu_n * k)
    out["cfg5_fp16_decode_fwd_M16_K8192_N28672"] = {
        "gpu": {"us_p50": _r(t["p50"] * 1e3, 1), "us_p20": _r(t["p20"] * 1e3, 1), "us_p80": _r(t["p80"] * 1e3, 1),
                "bytes": nbytes, "gbps": _r(nbytes / t["p50"] / 1e6, 1), "tflops": _r(6.0 * m * n * k / t["p50"] / 1e9, 1),
                "cache_flush_between_reps": True,
                "roofline": {"bound": "hbm", "achieved": _r(nbytes / t["p50"] / 1e6, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                             "frac": _r(nbytes / t["p50"] / 1e6 / PEAK_HBM_GBPS), "traffic": traffic,
                             "traffic_source": traffic_src}},
        "cpu": {"ms": _r(cpu_t * 1e3, 1), "gbps": _r(3 * k * cpu_n * 4 / cpu_t / 1e9, 1), "tflops": _r(cpu_tf, 4),
                "sample": f"all 16 rows, intermediate columns 0..{cpu_n - 1} of {n} (fp32 weights: {3 * k * cpu_n * 4 / 1e6:.0f} MB), "
                          "fp32 torch-CPU oracle, median of 2 after 1 warm-up"},
    }
    del x, Wg, Wu, Wd
    return out


def _edge_shapes(dev):
    """Shapes off the tile grid, next to torch's own operators (rocBLAS/hipBLASLt) on the same GPU:
    a ragged token count at the headline widths (fwd+bwd), a short batch at the decode widths
    (forward; the down projection splits its reduction), a batch of one and a half rounds of tiles
    (stream-K) and a batch whose 2.3 GB activations are beyond 32-bit byte offsets (fwd+bwd; the
    module runs it as two row chunks)."""
    from triton_gated_mlp import EagerGatedMLP, FusedGatedMLP, copy_weights

    out = {}
    for name, (m, k, n, bwd) in {
        "ragged_fp16_fwdbwd_M8191_K4096_N14336": (8191, 4096, 14336, True),
        "one_and_a_half_rounds_fp16_fwdbwd_M6144_K4096_N14336": (6144, 4096, 14336, True),
        "short_batch_fp16_fwd_M32_K8192_N28672": (32, 8192, 28672, False),
        "tall_batch_fp16_fwdbwd_M40960_K8192_N28672": (40960, 8192, 28672, True),
    }.items():
        fused = FusedGatedMLP(hidden_size=k, intermediate_size=n, bias=False).to(dev).to(DTYPE)
        eager = EagerGatedMLP(hidden_size=k, intermediate_size=n, bias=False).to(dev).to(DTYPE)
        x, dy = _stated_inputs(fused, m, k, dev, DTYPE, bwd)
        copy_weights(fused, eager)
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

            big = m > 8192
            res[label] = _r(_bench(step, warmup_ms=0.0 if big else 25.0, rep_ms=0.0 if big else 60.0, min_reps=3 if big else 5)["p50"])
        flop = (18.0 if bwd else 6.0) * m * n * k
        res["tflops"] = _r(flop / res["ms"] / 1e9, 1)
        out[name] = res
        del fused, eager, x, dy
    return out


def _cpu_baseline():
    """CPU oracle on a bounded sample of the headline workload: the first 2048 of the 8192 token rows,
    same K and N, forward+backward."""
    ms = 2048
    t, tf = _cpu_leg(ms, K, N, True, False, 0.0, 18.0 * N * K)
    info = _cpu_info()
    return {"value": _r(tf), "unit": "TFLOP/s", "cores": info["cores"], "kind": "port",
            "sample": f"fwd+bwd of rows 0..{ms - 1} of the workload (M={ms}, K={K}, N={N}), fp32 torch-CPU oracle, "
                      f"median of 2 after 1 warm-up, {t * 1e3:.0f} ms/step",
            "os_cpu_count": info["os_cpu_count"], "cpu_model": info["cpu_model"]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip per-kernel breakdown, other configurations and edge shapes")
    ap.add_argument("--step-only", action="store_true",
                    help="time the steps and nothing else (no roofline launch, quantiles, extras or CPU leg): what a kernel "
                         "trace of the step itself is taken from")
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

    if args.step_only:
        print(json.dumps({"metric": "fwd+bwd TFLOP/s & % MFMA peak, fp16 M=8192 K=4096 N=14336 (1 GPU)", "value": round(tflops, 2),
                          "unit": "TFLOP/s", "ms_per_step": round(ms_per_step, 4), "steps": args.steps, "warmup": args.warmup,
                          "note": "--step-only: the timed steps alone"}), flush=True)
        return

    # dominant launch: dW_gate, dW_up and dW_down through gmlp_dw_bwd_grouped (6*M*N*K FLOP): one grid
    # of whole rounds of tiles, the pieces of the last half round's tiles (stream-K) and their sums;
    # events on the launch stream around the three kernels
    from triton_gated_mlp.ops import bwd as B
    from triton_gated_mlp.ops import fwd as F

    Wg, Wu, Wd = mlp.gate_proj.weight.detach(), mlp.up_proj.weight.detach(), mlp.down_proj.weight.detach()
    xd = x.detach()
    hs = F.gateup_fwd(xd, Wg, None, Wu, None, save_activations=True)
    dg, du = B.dh_bwd(dY, Wd, hs.gate, hs.up)
    dw_call = lambda: B.dw_bwd_grouped([(dg, xd), (du, xd), (dY, hs.hidden)])
    # back to back (as the kernels run under rocprofv3 in profiles/) and behind a cache flush (as the
    # `kernels` block times every launch); inside a step the call sits between the two
    t = _bench(dw_call, rep_ms=60.0, min_reps=max(args.steps, 10), flush=False)
    t_flushed = _bench(dw_call, rep_ms=40.0, min_reps=10, flush=True)
    del dg, du, hs
    dom_flop = 6.0 * M * N * K
    traffic, traffic_src = _traffic_from_profile(DW_GROUP_TRAFFIC_PROFILE)
    roofline = dict(
        _mfma_block(dom_flop, t["mean"]),
        kernel="gmlp_dw_bwd_grouped (dW_gate + dW_up + dW_down): gemm_group_kernel_pipelined<f16,256,256,16,...,EpiStore> over 2560 "
               "tiles, gemm_kernel_pipelined<...,stream-K> over the pieces of the other 128, streamk_fixup_kernel",
        avg_launch_ms=_r(t["mean"]), p50_launch_ms=_r(t["p50"]), launches_timed=t["reps"], timing="HIP events on the launch stream, "
        "calls back to back, no cache flush", flushed_launch_ms=_r(t_flushed["mean"]), frac_flushed=_r(dom_flop / t_flushed["mean"] / 1e9 / PEAK_MFMA_F16_TFLOPS),
        flop_per_launch=dom_flop, traffic=traffic, algorithmic_bytes=DW_GROUP_ALGORITHMIC_BYTES, traffic_source=traffic_src,
    )

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
    q = _bench(step, rep_ms=100.0, min_reps=10)
    line["step_quantiles"] = {"ms_p50": _r(q["p50"]), "ms_p20": _r(q["p20"]), "ms_p80": _r(q["p80"]), "reps": q["reps"],
                              "cache_flush_between_reps": True, "tflops_p50": _r(flop_step / q["p50"] / 1e9, 1)}
    if not args.no_extras:
        line["kernels"] = _kernel_breakdown(mlp, x, dY)
    del mlp, x, dY, params
    if not args.no_extras:
        line["configs"] = _config_lines(dev)
        line["edge_shapes"] = _edge_shapes(dev)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = _cpu_baseline()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
