#!/usr/bin/env python3
"""The reference's benchmark sweep on the HIP path: one head, d = 64, fp16, N_Q = N_K = 8192 ... 2097152,
non-causal (``fhog/benchhhh.py:15-27,93-110``; its x axis is ``assets/speedup.png``).

    python flash-hob_amd/fhog/sweep.py [--max-n 2097152] [--dtype fp16|bf16] [--budget-ms 3000] [--schedule three_sweep]

Prints one line per size: milliseconds per call (median and minimum of the timed calls, the statistics of the
reference's ``do_bench``) and algorithmic TFLOP/s (24 * d * N^2 FLOP per call).  The time budget per size plays the
role of ``do_bench(rep=5000, warmup=300)``.  The reference draws O and L at random (timing only; exp(S - L) then
overflows for some rows); here they come from a forward pass on the same Q, K, V, so the timed call computes finite,
meaningful numbers.
"""
import argparse
import statistics
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

SIZES = [8192, 16384, 32768, 65536, 131072, 262144, 524288, 1048576, 2097152]
D = 64


def sweep_point(n, dtype, budget_ms=3000.0, max_calls=200, min_calls=3, fused_stats=False, device="cuda:0", schedule=None):
    """One size of the sweep: dict with ms (median), ms_min, calls and algorithmic TFLOP/s (from the median)."""
    import torch
    import fhog
    g = torch.Generator(device="cpu").manual_seed(n)
    mk = lambda std: (torch.randn(1, n, D, generator=g) * std).to(dtype).to(device)
    q, k, v = mk(1.0), mk(1.0), mk(1.0)
    do, ddq, ddk, ddv = mk(0.1), mk(0.1), mk(0.1), mk(0.1)
    scale = D ** -0.5
    o, L = fhog.attention_forward(q, k, v, scale, False)
    plan = fhog.BwdBwdPlan(q, k, v, o, do, ddq, ddk, ddv, L, scale, fused_stats=fused_stats, schedule=schedule)
    plan.run()
    torch.cuda.synchronize()
    times, spent = [], 0.0
    while len(times) < min_calls or (spent < budget_ms and len(times) < max_calls):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        plan.run()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
        spent += times[-1]
    ms = statistics.median(times)
    finite = all(bool(torch.isfinite(t.float()).all()) for t in plan.outs)
    return {"n": n, "ms": round(ms, 4), "ms_min": round(min(times), 4), "calls": len(times),
            "tflops": round(24 * D * n * n / ms / 1e9, 1), "finite": finite}


def main():
    import torch
    ap = argparse.ArgumentParser()
    ap.add_argument("--max-n", type=int, default=SIZES[-1])
    ap.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16")
    ap.add_argument("--budget-ms", type=float, default=3000.0, help="timed milliseconds per size (at least 3 calls)")
    ap.add_argument("--fused-stats", action="store_true")
    ap.add_argument("--schedule", default=None, help="one of the opt-in schedules of flash_bwdbwd (default: the reference's four passes)")
    args = ap.parse_args()
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    for n in [s for s in SIZES if s <= args.max_n]:
        r = sweep_point(n, dtype, args.budget_ms, fused_stats=args.fused_stats, schedule=args.schedule)
        print(f"N={n:8d} {args.dtype} d={D}: {r['ms']:10.3f} ms/call (min {r['ms_min']:.3f})  {r['tflops']:7.1f} TFLOP/s algorithmic "
              f"({r['calls']} calls, outputs finite: {r['finite']})", flush=True)


if __name__ == "__main__":
    main()
