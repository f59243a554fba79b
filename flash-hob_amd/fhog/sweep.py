#!/usr/bin/env python3
"""The reference's benchmark sweep on the HIP path: one head, d = 64, fp16, N_Q = N_K = 8192 ... 2097152,
non-causal, all nine tensors random (``fhog/benchhhh.py:15-110``; its x axis is ``assets/speedup.png``).

    python flash-hob_amd/fhog/sweep.py [--max-n 2097152] [--dtype fp16|bf16] [--budget-ms 3000]

Prints one line per size: milliseconds per call (median of the timed calls) and algorithmic TFLOP/s
(24 * d * N^2 FLOP per call).  The time budget per size plays the role of ``do_bench(rep=5000, warmup=300)``.
"""
import argparse
import statistics
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

SIZES = [8192, 16384, 32768, 65536, 131072, 262144, 524288, 1048576, 2097152]


def main():
    import torch
    import fhog
    ap = argparse.ArgumentParser()
    ap.add_argument("--max-n", type=int, default=SIZES[-1])
    ap.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16")
    ap.add_argument("--budget-ms", type=float, default=3000.0, help="timed milliseconds per size (at least 3 calls)")
    ap.add_argument("--fused-stats", action="store_true")
    args = ap.parse_args()
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    dev = torch.device("cuda:0")
    d = 64
    for n in [s for s in SIZES if s <= args.max_n]:
        g = torch.Generator(device="cpu").manual_seed(n)
        mk = lambda *shape: torch.randn(*shape, generator=g).to(dtype).to(dev)
        q, k, v, o, do, ddq, ddk, ddv = (mk(1, n, d) for _ in range(8))
        L = mk(1, n)
        plan = fhog.BwdBwdPlan(q, k, v, o, do, ddq, ddk, ddv, L, d ** -0.5, fused_stats=args.fused_stats)
        plan.run()
        torch.cuda.synchronize()
        times, spent = [], 0.0
        while len(times) < 3 or spent < args.budget_ms:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            plan.run()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1))
            spent += times[-1]
            if len(times) >= 200:
                break
        ms = statistics.median(times)
        print(f"N={n:8d} {args.dtype} d={d}: {ms:10.3f} ms/call  {24 * d * n * n / ms / 1e9:7.1f} TFLOP/s algorithmic "
              f"({len(times)} calls)", flush=True)


if __name__ == "__main__":
    main()
