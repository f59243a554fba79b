#!/usr/bin/env python3
"""Headline benchmark: attention double-backward on one MI355X.

One "step" = one call of ``fhog.flash_bwdbwd`` (the reference's four passes dd, b, dQ'+ddO, dK'+dV'; the first also writes d) on
seeded synthetic tensors that are already resident in HBM.  The workload is the configuration the
metric is quoted on: bf16 causal B=2 H=16 N=4096 d=128.

Prints ONE JSON line.  ``value`` is the whole-path algorithmic throughput
(24*d*pairs FLOP per step: the 12 contractions of the materialised formula, recomputation
not counted).  ``roofline`` describes the dominant kernel (pass 3, dQ'+ddO) against the dense
bf16 MFMA peak; ``cpu_baseline`` is the torch autograd double-backward timed on this box's
host cores on a few heads of the same workload.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (ROOT / "flash-hob_amd", ROOT):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))

PEAK_BF16_TFLOPS = 2516.6   # MI355X dense bf16 MFMA: 256 CU x 4096 FLOP/clk x 2.4 GHz
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PASS_NAMES = {0: "rowdot_kernel (not in the 16-bit chain: its pass 1 writes d too)", 1: "q_sweep_bf16<pass 1: d, dd>",
              2: "q_sweep_bf16<pass 2: b>",
              3: "q_sweep3_pc<pass 3: dQ2, ddO>", 4: "k_sweep_pc<pass 4: dK2, dV2>",
              5: "q_sweep_bf16<fused passes 1+2: d, dd, b> (opt-in schedule)",
              6: "q_sweep_ddo<pass 6: b, ddO from dd> (opt-in schedule)",
              7: "q_sweep3_pc<pass 7: dQ2 alone> (opt-in schedules)",
              8: "q_sweep_ddo<pass 8: d, dd, b, ddO> (opt-in schedule)"}
# contractions each kernel needs to produce its outputs from its inputs (2*d*pairs FLOP each)
PASS_CONTRACTIONS = {0: 0, 1: 3, 2: 5, 3: 9, 4: 8, 5: 5, 6: 5, 7: 7, 8: 5}
# recomputed products of each schedule of the 16-bit family (the materialised formula has 12)
SCHEDULE_PRODUCTS = {"four_pass": 25, "fused_stats": 22, "ddo_early": 23, "three_sweep": 20}


def event_times_ms(fn, iters):
    """Time `iters` calls of fn on torch's current stream (the stream the library's kernels are launched on), one event
    between every two calls. Returns mean (first event to last: exactly `iters` calls between two synchronisations),
    median and minimum of the per-call intervals, as the reference's do_bench reports them (fhog/benchhhh.py:58,76)."""
    import statistics
    import torch
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
    torch.cuda.synchronize()
    ev[0].record()
    for i in range(iters):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    each = [ev[i].elapsed_time(ev[i + 1]) for i in range(iters)]
    return {"mean": ev[0].elapsed_time(ev[iters]) / iters, "median": statistics.median(each), "min": min(each)}


def event_time_ms(fn, iters):
    return event_times_ms(fn, iters)["mean"]


def mfma_sustained(dev, trips=20000, repeats=2):
    """bf16 MFMA rate of a loop of nothing but MFMAs, on zero and on random operands (TFLOP/s): the rate the chip holds
    under its power limit depends on the operand data; the second figure is the practical ceiling for real tensors."""
    import ctypes
    import torch
    from fhog import _lib
    L = _lib.lib()
    blocks = torch.cuda.get_device_properties(dev).multi_processor_count
    out = torch.empty(blocks * 512, dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = {}
    # the last three: the same random-operand loop with the A operands read from LDS (one 128-bit read per MFMA,
    # prefetched: the matrix pipe never waits for them), with three VALU instructions per MFMA, and with both - what
    # the power limit leaves of the MFMA rate for a kernel with the instruction mix of the recomputation sweeps
    # the last: modes 1, 2, 4 with ONE wave per SIMD, where a wave's LDS reads and VALU instructions have only its own MFMAs
    # to hide behind: what they cost a wave in issue time (the figures above are what they cost in clock)
    for name, mode in (("zeros", 0), ("random", 1), ("random_lds_read_per_mfma", 2), ("random_lds_read_per_2_mfma", 3),
                       ("random_3_valu_per_mfma", 4), ("random_lds_read_and_3_valu_per_mfma", 5),
                       ("one_wave_per_simd_random", 9), ("one_wave_per_simd_lds_read_per_mfma", 10),
                       ("one_wave_per_simd_3_valu_per_mfma", 12), ("one_wave_per_simd_lds_read_and_3_valu_per_mfma", 13)):
        flops = ctypes.c_double()
        run = lambda trips: _lib.check(L.fhog_probe_mfma_rate(out.data_ptr(), blocks, trips, mode, ctypes.byref(flops), stream))
        run(trips)   # warm-up, also lets the clock settle
        ms = event_time_ms(lambda: run(trips), repeats)
        res[name] = round(flops.value / ms / 1e9, 1)
    return res


def other_workloads(dev, skip):
    """The remaining reference configurations (parity-test cases, not the headline): ms per call and algorithmic TFLOP/s
    of the same entry point, default schedule, caches from the HIP forward where it applies."""
    import torch
    import fhog
    from fhog.workloads import WORKLOADS, make_inputs
    res = {}
    for name, w in WORKLOADS.items():
        if name == skip:
            continue
        x = {n: t.flatten(0, 1).to(dev) for n, t in make_inputs(w, seed=0).items()}
        o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], w.scale, w.causal)
        plan = fhog.BwdBwdPlan(x["Q"], x["K"], x["V"], o, x["dO"], x["ddQ"], x["ddK"], x["ddV"], L, w.scale, causal=w.causal)
        for _ in range(10):   # the host spent seconds making the inputs: let the clocks come back up
            plan.run()
        ms = event_time_ms(plan.run, 20 if w.flops_algorithmic < 2e12 else 5)
        tflops = w.flops_algorithmic / ms / 1e9
        fp32 = plan.impl == 1
        res[name] = {"ms_per_step_no_alloc": round(ms, 4), "value": round(tflops, 2),
                     "kernel_family": "fp32-mfma" if fp32 else "bf16-mfma",
                     # against the peak of the matrix instructions the workload runs on
                     ("pct_fp32_mfma_peak" if fp32 else "pct_bf16_mfma_peak"):
                         round(100 * tflops / (PEAK_FP32_TFLOPS if fp32 else PEAK_BF16_TFLOPS), 2)}
        del x, o, L, plan
        torch.cuda.empty_cache()
    return res


def first_order(w, x, iters):
    """The callers on either side of the path on the same workload: HIP forward (O, L) and HIP first backward
    (dQ, dK, dV). FLOP counts: 2 products forward, 5 backward (the kernels recompute S and dP once per direction: 7)."""
    import fhog
    if w.d not in (64, 128) or w.dtype.itemsize != 2:
        return None
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], w.scale, w.causal)
    fwd = event_time_ms(lambda: fhog.attention_forward(x["Q"], x["K"], x["V"], w.scale, w.causal), iters)
    bwd = event_time_ms(lambda: fhog.attention_backward(x["Q"], x["K"], x["V"], o, x["dO"], L, w.scale, w.causal), iters)
    unit = 2 * w.d * w.pairs
    res = {"forward_ms": round(fwd, 4), "forward_tflops": round(2 * unit / fwd / 1e9, 1),
           "backward_ms": round(bwd, 4), "backward_tflops": round(5 * unit / bwd / 1e9, 1),
           "note": "fhog_attn_fwd / fhog_attn_bwd including output allocation; not part of `value`"}
    # the fp32-MFMA first-order kernels at their largest head dim (fp32 tensors, causal, 32 slices of 2048 tokens)
    import torch
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (torch.randn(32, 2048, 128, generator=g).to(x["Q"].device) for _ in range(4))
    scale, pairs = 128 ** -0.5, 32 * 2048 * 2049 // 2
    o32, L32 = fhog.attention_forward(q, k, v, scale, True, use_hip=True)
    f32 = event_time_ms(lambda: fhog.attention_forward(q, k, v, scale, True, use_hip=True), 5)
    b32 = event_time_ms(lambda: fhog.attention_backward(q, k, v, o32, do, L32, scale, True, use_hip=True), 5)
    res["fp32_d128_causal_2048"] = {"forward_ms": round(f32, 4), "forward_tflops": round(2 * 2 * 128 * pairs / f32 / 1e9, 1),
                                    "backward_ms": round(b32, 4), "backward_tflops": round(5 * 2 * 128 * pairs / b32 / 1e9, 1),
                                    "peak": PEAK_FP32_TFLOPS}
    return res


def reference_sweep(max_n=65536):
    """The first sizes of the reference's own benchmark sweep (fhog/benchhhh.py:15-27,93-110: one head, d = 64, fp16,
    non-causal, N = 8192, 16384, ...; the x axis of assets/speedup.png): ms per call (median, min) and algorithmic
    TFLOP/s. The whole list, up to N = 2097152, is `python flash-hob_amd/fhog/sweep.py`."""
    import torch
    from fhog.sweep import SIZES, sweep_point
    return {"dtype": "f16", "d": 64, "heads": 1, "causal": False,
            "points": [sweep_point(n, torch.float16, budget_ms=150.0, max_calls=30, min_calls=5) for n in SIZES if n <= max_n]}


def traffic_bytes(workload, pass_id):
    """HBM bytes per launch of one pass from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised under
    profiles/ (the summary carries them in a machine-readable comment, written by fhog/rocprof_summary.py);
    None when that workload or pass has no measurement."""
    import re
    for f in sorted((ROOT / "profiles").glob(f"bwdbwd_kernels_{workload}*.md")):
        m = re.search(r"<!-- traffic_bytes: (\{.*?\}) -->", f.read_text())
        if m:
            return json.loads(m.group(1)).get(str(pass_id))
    return None


def cpu_baseline(w, x_cpu, heads, repeats):
    """torch autograd double-backward (fp32, materialised, one head at a time) on the host cores."""
    import torch
    from oracle.bwdbwd_oracle import autograd_double_backward
    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))))
    sel = {n: t[:heads].float() for n, t in x_cpu.items()}
    args = (sel["Q"], sel["K"], sel["V"], sel["dO"], sel["ddQ"], sel["ddK"], sel["ddV"], w.scale, w.causal)
    autograd_double_backward(*(a[:1] if torch.is_tensor(a) else a for a in args), dtype=torch.float32)  # warm-up, 1 head
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        autograd_double_backward(*args, dtype=torch.float32)
        best = min(best, time.perf_counter() - t0)
    flops = w.flops_algorithmic * heads / w.batch
    return {"value": round(flops / best / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{heads} of {w.batch} (batch*head) slices of {w.name}, fp32 torch autograd double-backward on "
                      f"materialised attention, best of {repeats}, {best:.2f} s",
            "seconds": round(best, 3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None, help="one of fhog.workloads.WORKLOADS (default: the headline)")
    ap.add_argument("--cpu-heads", type=int, default=32, help="slices of the workload timed on the CPU (0 = skip)")
    ap.add_argument("--profile-only", action="store_true", help="run the timed loop only (for rocprofv3)")
    ap.add_argument("--probe-only", action="store_true", help="run the MFMA rate probes only and print their figures (for rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU (the path shards over batch*head with no communication); "
                 "run with --gpus 1")

    import torch
    import fhog
    from fhog.workloads import HEADLINE, WORKLOADS, make_inputs
    from fhog import _lib
    assert torch.cuda.is_available(), "bench.py needs a ROCm GPU"
    _lib.lib()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    if args.probe_only:
        print(json.dumps(mfma_sustained(dev, trips=20000, repeats=3)))
        return
    w = WORKLOADS[args.workload or HEADLINE]

    x_cpu = {n: t.flatten(0, 1) for n, t in make_inputs(w, seed=0).items()}
    x = {n: t.to(dev) for n, t in x_cpu.items()}
    o, L = fhog.attention_forward(x["Q"], x["K"], x["V"], w.scale, w.causal, use_hip=False)   # caches (fp32 forward); not timed
    call = lambda: fhog.flash_bwdbwd(x["Q"], x["K"], x["V"], o, x["dO"], x["ddQ"], x["ddK"], x["ddV"], L, w.scale,
                                     causal=w.causal)

    base_inputs = torch.cuda.memory_allocated()   # the eight inputs, O and L (the plans' own outputs come on top)
    plan = fhog.BwdBwdPlan(x["Q"], x["K"], x["V"], o, x["dO"], x["ddQ"], x["ddK"], x["ddV"], L, w.scale, causal=w.causal)

    def headline():
        """W untimed calls, then exactly K timed calls of the drop-in entry point (allocation of outputs and workspace
        included), and the memory they take on top of what is resident."""
        for _ in range(args.warmup):
            call()
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base_mem = torch.cuda.memory_allocated()
        t = event_times_ms(call, args.steps)
        return t, torch.cuda.max_memory_allocated() - base_mem

    if args.profile_only:
        headline()
        fused = fhog.BwdBwdPlan(x["Q"], x["K"], x["V"], o, x["dO"], x["ddQ"], x["ddK"], x["ddV"], L, w.scale,
                                causal=w.causal, fused_stats=True)
        for _ in range(3):
            fused.run()   # the opt-in fused statistics sweep, so that it shows in the same trace
        for name in ("ddo_early", "three_sweep"):   # ... and the schedules that take ddO out of the third sweep
            alt = fhog.BwdBwdPlan(x["Q"], x["K"], x["V"], o, x["dO"], x["ddQ"], x["ddK"], x["ddV"], L, w.scale, causal=w.causal,
                                  schedule=name)
            for _ in range(3):
                alt.run()
        for _ in range(3):  # the first-order kernels (HIP forward and first backward) on the same tensors
            o16, L16 = fhog.attention_forward(x["Q"], x["K"], x["V"], w.scale, w.causal)
            fhog.attention_backward(x["Q"], x["K"], x["V"], o16, x["dO"], L16, w.scale, w.causal)
        # a plain streaming kernel of known size (reads 256 MiB, writes 256 MiB) to calibrate byte counters
        src = torch.zeros(64 * 2 ** 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        return

    # The secondary figures come first: the host spent seconds generating the inputs, and the GPU's clock governor
    # needs about 20 ms of load to leave its idle state (the first calls after an idle period run 3-10 % slower, whoever
    # issues them). The headline region then runs in the state a training loop is in.
    for _ in range(max(args.warmup, 40)):
        plan.run()
    t_plan = event_times_ms(plan.run, args.steps)
    ms_plan = t_plan["mean"]
    t_pass = {}
    for i in PASS_NAMES:
        plan.run(only_pass=i)   # untimed: the first launch of a kernel loads its code and raises its LDS limit
        t_pass[i] = event_times_ms(lambda i=i: plan.run(only_pass=i), args.steps)
    per_pass = {i: t["mean"] for i, t in t_pass.items()}
    dom = max((i for i in per_pass if i <= 4), key=PASS_CONTRACTIONS.get)   # the kernel of the default schedule with the largest share of the work
    opt_in = {}
    for name in ("fused_stats", "ddo_early", "three_sweep"):
        alt = fhog.BwdBwdPlan(x["Q"], x["K"], x["V"], o, x["dO"], x["ddQ"], x["ddK"], x["ddV"], L, w.scale, causal=w.causal,
                              schedule=name)
        alt.run()               # untimed first launch of the schedule's own kernels
        t_alt = event_time_ms(alt.run, args.steps)
        v_alt = w.flops_algorithmic / t_alt / 1e9
        opt_in[name] = {"ms_per_step_no_alloc": round(t_alt, 4), "value": round(v_alt, 2),
                        "pct_bf16_mfma_peak": round(100 * v_alt / PEAK_BF16_TFLOPS, 2),
                        "recomputed_products": SCHEDULE_PRODUCTS[name]}
        del alt
    ms_fused = opt_in["fused_stats"]["ms_per_step_no_alloc"]
    t_call, peak_extra = headline()
    ms = t_call["mean"]
    peak_total = base_inputs + peak_extra
    dom_flops = 2 * w.d * w.pairs * PASS_CONTRACTIONS[dom]
    dom_tflops = dom_flops / per_pass[dom] / 1e9

    value = w.flops_algorithmic / ms / 1e9
    out = {
        "metric": "double-bwd TFLOP/s, % bf16 MFMA peak @B2 H16 N4096 d128 causal; peak mem GB",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "ms_per_step_median": round(t_call["median"], 4),
        "ms_per_step_min": round(t_call["min"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {"workload": w.name, "B": w.B, "H": w.H, "n_q": w.n_q, "n_k": w.n_k, "d": w.d, "causal": w.causal,
                   "seed": 0, "kernel_family": {1: "fp32-mfma", 2: "bf16-mfma"}[plan.impl]},
        "pct_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
        "executed_tflops": round(w.flops_executed / ms / 1e9, 2),
        "peak_mem_gb": round(peak_total / 1e9, 4),
        "peak_mem_call_gb": round(peak_extra / 1e9, 4),
        "ms_per_step_no_alloc": round(ms_plan, 4),
        "ms_per_step_no_alloc_median": round(t_plan["median"], 4),
        "ms_per_step_no_alloc_min": round(t_plan["min"], 4),
        "fused_stats_schedule": {"ms_per_step_no_alloc": round(ms_fused, 4),
                                 "value": round(w.flops_algorithmic / ms_fused / 1e9, 2),
                                 "note": "opt-in: dd and b from one sweep (22 recomputed products instead of 25)"},
        # every opt-in schedule on the same tensors (same algorithmic FLOP count, fewer recomputed products); `value`
        # above is the reference's four-pass schedule (25)
        "opt_in_schedules": opt_in,
        "ms_per_pass": {PASS_NAMES[i]: round(t, 4) for i, t in per_pass.items()},
        "ms_per_pass_median_min": {PASS_NAMES[i]: [round(t["median"], 4), round(t["min"], 4)] for i, t in t_pass.items()},
        "roofline": {"bound": "mfma", "kernel": PASS_NAMES[dom], "achieved": round(dom_tflops, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(dom_tflops / PEAK_BF16_TFLOPS, 4),
                     # whole path: the 12 products of the materialised formula over the time of one call, against the peak
                     "frac_algorithmic": round(value / PEAK_BF16_TFLOPS, 4),
                     "flops_per_launch": dom_flops, "ms_per_launch": round(per_pass[dom], 4),
                     "ms_per_launch_median": round(t_pass[dom]["median"], 4), "traffic": traffic_bytes(w.name, dom)},
    }
    if not args.workload:
        out["other_workloads"] = other_workloads(dev, skip=w.name)
        out["reference_sweep"] = reference_sweep()
    fo = first_order(w, x, min(args.steps, 20))
    if fo:
        out["first_order"] = fo
    out["mfma_sustained_tflops"] = mfma_sustained(dev)
    out["roofline"]["frac_of_sustained_random"] = round(dom_tflops / out["mfma_sustained_tflops"]["random"], 4)
    # What a loop of nothing but MFMAs on random operands would leave of the algorithmic figure under the four-pass
    # schedule, which issues 25 products for the 12 it is credited with: the ceiling of `value` on this box.
    sustained = out["mfma_sustained_tflops"]["random"]
    # ... and the same for a loop that also carries one LDS operand read and three VALU instructions per MFMA, the
    # instruction mix of the sweeps (still nothing the matrix pipe waits for: profiles/mfma_rate_instruction_mix.md)
    mix = out["mfma_sustained_tflops"]["random_lds_read_and_3_valu_per_mfma"]
    out["ceiling"] = {"sustained_random_tflops": sustained,
                      "four_pass_algorithmic_tflops": round(sustained * 12 / 25, 1),
                      "pct_of_ceiling": round(100 * value / (sustained * 12 / 25), 2),
                      "sustained_random_with_sweep_instruction_mix_tflops": mix,
                      "four_pass_algorithmic_with_mix_tflops": round(mix * 12 / 25, 1),
                      "pct_of_ceiling_with_mix": round(100 * value / (mix * 12 / 25), 2)}
    if args.cpu_heads > 0:
        out["cpu_baseline"] = cpu_baseline(w, x_cpu, min(args.cpu_heads, w.batch), repeats=2)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
