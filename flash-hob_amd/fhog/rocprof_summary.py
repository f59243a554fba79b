#!/usr/bin/env python3
"""Turn the raw output of four rocprofv3 runs of ``bench.py --profile-only`` into the short summary kept under
``profiles/``: per-kernel time, HBM bytes per launch (FETCH_SIZE / WRITE_SIZE, calibrated on a streaming kernel of known
size) and the SQ counters behind the matrix-pipe occupancy.

    cd /tmp && export TMPDIR=/tmp && cd <repo>
    W=cfg2_bf16_causal_4096_d128; OUT=prof_out        # any scratch directory
    rocprofv3 --kernel-trace --stats -d $OUT/prof_kt -o kt --output-format csv -- python3 bench.py --profile-only --workload $W --steps 20 --warmup 5
    rocprofv3 --pmc FETCH_SIZE -d $OUT/prof_fetch -o f --output-format csv -- python3 bench.py --profile-only --workload $W --steps 3 --warmup 1
    rocprofv3 --pmc WRITE_SIZE -d $OUT/prof_write -o w --output-format csv -- python3 bench.py --profile-only --workload $W --steps 3 --warmup 1
    rocprofv3 --pmc SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_VALU_MFMA_COEXEC_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_LDS_IDX_ACTIVE SQ_LDS_BANK_CONFLICT -d $OUT/prof_sq -o s --output-format csv -- python3 bench.py --profile-only --workload $W --steps 3 --warmup 1
    python3 flash-hob_amd/fhog/rocprof_summary.py --workload $W --root $OUT > profiles/bwdbwd_kernels_$W.md

``bench.py`` reads the HBM bytes of the dominant kernel back from the machine-readable comment this script writes.
"""
import argparse
import collections
import csv
import json
import re
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

COMMANDS = __doc__.split("cd <repo>\n")[1].split("\n\n``bench.py``")[0]


def short(name):
    k = name.replace("void fhog::(anonymous namespace)::", "").replace("(fhog::Params)", "").replace("(fhog::AttnParams)", "")
    if "rowdot" in k:
        k = "rowdot_kernel"
    return k


def pass_of(kernel):
    """Pass id of a double-backward kernel (fhog_hip.h), 'fwd' / 'bwd_q' / 'bwd_k' for the first-order ones, else None."""
    m = re.match(r"q_sweep_bf16<\w+, \d+, (\d)", kernel)
    if m:
        return int(m.group(1))
    m = re.match(r"q_sweep_ddo<\w+, \d+, \d, (\w+)[,>]", kernel)
    if m:
        return 6 if m.group(1) == "true" else 8
    if re.match(r"q_sweep3_pc<\w+, \d+, \d, true>", kernel):
        return 7
    for prefix, p in (("dd_sweep64_bf16", 1), ("q_stage1_bf16", 9), ("q_sweep3_pc", 3), ("k_sweep_pc", 4), ("k_sweep_bf16", 4), ("rowdot", 0), ("attn_fwd", "fwd"),
                      ("attn_bwd_q", "bwd_q"), ("attn_bwd_k", "bwd_k")):
        if kernel.startswith(prefix):
            return p
    return None


def algorithmic_mib(w, p):
    """(read, written) MiB one launch of pass p has to move: every input once, every output once."""
    es = w.dtype.itemsize
    qt, kt, rv = w.batch * w.n_q * w.d * es / 2 ** 20, w.batch * w.n_k * w.d * es / 2 ** 20, w.batch * w.n_q * 4 / 2 ** 20
    table = {0: (2 * qt, rv), 1: (4 * qt + 2 * kt + rv, 2 * rv), 2: (3 * qt + 4 * kt + 3 * rv, rv),
             5: (4 * qt + 4 * kt + rv, 3 * rv), 6: (3 * qt + 4 * kt + 3 * rv, qt + rv), 7: (3 * qt + 4 * kt + 4 * rv, qt),
             8: (4 * qt + 4 * kt + rv, qt + 3 * rv), 9: (4 * qt + 4 * kt + rv, 2 * qt + 3 * rv), 3: (3 * qt + 4 * kt + 4 * rv, 2 * qt), 4: (3 * qt + 4 * kt + 4 * rv, 2 * kt),
             "fwd": (qt + 2 * kt, qt + rv), "bwd_q": (2 * qt + 2 * kt + 2 * rv, qt), "bwd_k": (2 * qt + 2 * kt + 2 * rv, 2 * kt)}
    return table.get(p)


def counters(path):
    """{kernel: {counter: mean value per dispatch}}; 'calib' = the last three dispatches of the streaming torch.add."""
    a = collections.defaultdict(lambda: collections.defaultdict(list))
    for r in csv.DictReader(open(path)):
        k = r["Kernel_Name"]
        if "fhog" in k:
            a[short(k)][r["Counter_Name"]].append(float(r["Counter_Value"]))
        elif "elementwise" in k:
            a["calib"][r["Counter_Name"]].append(float(r["Counter_Value"]))
    for c in a.get("calib", {}):
        a["calib"][c] = a["calib"][c][-3:]
    return {k: {c: sum(v) / len(v) for c, v in d.items()} for k, d in a.items()}


def compare(w, variants):
    """One table row per (variant, double-backward kernel): average duration, matrix-pipe occupancy, clock, HBM bytes read.
    `variants`: list of (label, directory holding prof_kt, prof_fetch, prof_sq of a run made under that FHOG_TUNE)."""
    P = print
    P("| FHOG_TUNE | kernel | calls | avg ns | MFMA busy fraction | VALU per MFMA | clock GHz | HBM read MiB | HBM read / algorithmic |")
    P("|---|---|---|---|---|---|---|---|---|")
    for label, root in variants:
        root = Path(root)
        kt = {short(r["Name"]): r for r in csv.DictReader(open(root / "prof_kt" / "kt_kernel_stats.csv")) if "fhog" in r["Name"]}
        fe = counters(root / "prof_fetch" / "f_counter_collection.csv")
        sq = counters(root / "prof_sq" / "s_counter_collection.csv")
        sf = 262144 / fe["calib"]["FETCH_SIZE"]
        for k in sorted(kt, key=lambda k: str(pass_of(k))):
            p = pass_of(k)
            if not isinstance(p, int) or p == 0 or k not in sq or int(kt[k]["Calls"]) < 4:
                continue
            d = sq[k]
            cyc, ns = d["SQ_BUSY_CYCLES"] / 32, float(kt[k]["AverageNs"])
            f = fe[k]["FETCH_SIZE"] * sf / 1024
            P(f"| {label} | {k} | {kt[k]['Calls']} | {ns:.0f} | {d['SQ_VALU_MFMA_BUSY_CYCLES'] / 1024 / cyc:.3f} | "
              f"{(d['SQ_INSTS_VALU'] - d['SQ_INSTS_MFMA']) / d['SQ_INSTS_MFMA']:.2f} | {cyc / ns:.2f} | {f:.1f} | "
              f"{f / algorithmic_mib(w, p)[0]:.2f} |")


PROBE_MODES = {0: "operands all zero", 1: "random operands, nothing but MFMAs",
               2: "random, one LDS operand read (ds_read_b128) per MFMA", 3: "random, one LDS operand read per two MFMAs",
               4: "random, three v_fma_f32 per MFMA", 5: "random, one LDS read and three v_fma_f32 per MFMA"}


def probe_table(root, trips=20000, blocks=256):
    """The MFMA rate probes of `bench.py --probe-only`: rate, matrix-pipe occupancy and clock per instruction mix and
    number of waves per SIMD (kernel `mfma_rate_kernel<mode, waves per workgroup>`)."""
    root = Path(root)
    kt = {short(r["Name"]): r for r in csv.DictReader(open(root / "prof_kt" / "kt_kernel_stats.csv")) if "mfma_rate_kernel" in r["Name"]}
    sq = counters(root / "prof_sq" / "s_counter_collection.csv")
    P = print
    P("| mode | waves per SIMD | instruction mix | calls | avg ns | MFMA TFLOP/s | MFMA busy fraction | clock GHz | busy x clock | "
      "cycles per MFMA and wave | LDS active fraction |")
    P("|---|---|---|---|---|---|---|---|---|---|---|")
    for waves in (8, 4):
        for mode in sorted(PROBE_MODES):
            k = f"mfma_rate_kernel<{mode}, {waves}>(float*, int)"
            if k not in kt or k not in sq:
                continue
            flops = blocks * float(waves) * trips * 32 * 32768
            ns, d = float(kt[k]["AverageNs"]), sq[k]
            cyc = d["SQ_BUSY_CYCLES"] / 32
            busy = d["SQ_VALU_MFMA_BUSY_CYCLES"] / 1024 / cyc
            P(f"| {mode + (8 if waves == 4 else 0)} | {waves // 4} | {PROBE_MODES[mode]} | {kt[k]['Calls']} | {ns:.0f} | {flops / ns / 1e3:.0f} | "
              f"{busy:.3f} | {cyc / ns:.2f} | {busy * cyc / ns:.2f} | {cyc / (trips * 32):.1f} | {d['SQ_LDS_IDX_ACTIVE'] / 256 / cyc:.3f} |")


def main():
    from fhog.workloads import WORKLOADS
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default=None)
    ap.add_argument("--probe", metavar="DIR", help="instead of a summary: the table of the MFMA rate probes (DIR holds prof_kt and "
                    "prof_sq of `bench.py --probe-only`)")
    ap.add_argument("--root", default="prof_out", help="directory holding prof_kt, prof_fetch, prof_write, prof_sq")
    ap.add_argument("--note", default="", help="free text appended to the summary")
    ap.add_argument("--compare", nargs="+", metavar="LABEL@DIR", help="instead of a summary: one table over runs made under "
                    "different FHOG_TUNE settings (each DIR holds prof_kt, prof_fetch, prof_sq)")
    args = ap.parse_args()
    if args.probe:
        return probe_table(args.probe)
    w = WORKLOADS[args.workload]
    if args.compare:
        return compare(w, [tuple(c.rsplit("@", 1)) for c in args.compare])
    root = Path(args.root)
    kt = {short(r["Name"]): r for r in csv.DictReader(open(root / "prof_kt" / "kt_kernel_stats.csv")) if "fhog" in r["Name"]}
    fe = counters(root / "prof_fetch" / "f_counter_collection.csv")
    wr = counters(root / "prof_write" / "w_counter_collection.csv")
    sq = counters(root / "prof_sq" / "s_counter_collection.csv")
    order = sorted(kt, key=lambda k: -float(kt[k]["TotalDurationNs"]) if "TotalDurationNs" in kt[k] else -float(kt[k]["Percentage"]))
    P = print
    P(f"# rocprofv3 summary: double-backward kernels, workload {w.name} (B={w.B} H={w.H} N_Q={w.n_q} N_K={w.n_k} d={w.d} "
      f"{'causal' if w.causal else 'non-causal'} {str(w.dtype).replace('torch.', '')})\n")
    P("Commands (from the repository root on one MI355X):\n")
    P(COMMANDS.replace("W=cfg2_bf16_causal_4096_d128", f"W={w.name}"))
    P("""
`bench.py --profile-only` runs the timed loop of the default four-pass schedule, then three calls each of the opt-in
schedules (fused statistics: pass 5 replaces passes 1 and 2; ddO early: `q_sweep_ddo<.., true>` = pass 6 and
`q_sweep3_pc<.., true>` = pass 7 replace passes 2 and 3; three sweeps: `q_sweep_ddo<.., false>` = pass 8, then pass 7),
then three calls of the first-order kernels on the same tensors, then a streaming `torch.add` used to calibrate the byte
counters. Template arguments of the kernels: `<fp16?, d, [pass,] mask mode[, waves per workgroup | variant]>` (mask mode
1 = square causal mask).

## kernel-trace --stats (kt_kernel_stats.csv), library kernels only

| kernel | calls | avg ns | min ns | max ns | % of GPU time in the run |
|---|---|---|---|---|---|""")
    for k in order:
        r = kt[k]
        P(f"| {k} | {r['Calls']} | {float(r['AverageNs']):.0f} | {r['MinNs']} | {r['MaxNs']} | {float(r['Percentage']):.2f} |")
    cf, cw = fe["calib"]["FETCH_SIZE"], wr["calib"]["WRITE_SIZE"]
    sf, sw = 262144 / cf, 262144 / cw
    P(f"""
## HBM traffic per dispatch (--pmc FETCH_SIZE / WRITE_SIZE, KiB)

Calibration: the streaming kernel `torch.add(src, 1.0, out=dst)` on 64 Mi floats reads 262144 KiB and writes 262144 KiB;
the counters read FETCH_SIZE={cf:.1f}, WRITE_SIZE={cw:.1f} -> scale factors {sf:.3f} (fetch) and {sw:.3f} (write).

| kernel | FETCH_SIZE raw | WRITE_SIZE raw | HBM read MiB (scaled) | HBM write MiB (scaled) | algorithmic MiB (read + write) | HBM / algorithmic |
|---|---|---|---|---|---|---|""")
    traffic = {}
    for k in order:
        if k not in fe or k not in wr:
            continue
        f, wv = fe[k]["FETCH_SIZE"] * sf / 1024, wr[k]["WRITE_SIZE"] * sw / 1024
        alg = algorithmic_mib(w, pass_of(k))
        ratio = f"{(f + wv) / sum(alg):.2f}" if alg else ""
        alg_s = f"{alg[0]:.1f} + {alg[1]:.1f}" if alg else ""
        P(f"| {k} | {fe[k]['FETCH_SIZE']:.1f} | {wr[k]['WRITE_SIZE']:.1f} | {f:.1f} | {wv:.1f} | {alg_s} | {ratio} |")
        if isinstance(pass_of(k), int) and str(pass_of(k)) not in traffic:
            traffic[str(pass_of(k))] = int((f + wv) * 2 ** 20)
    P(f"\n<!-- traffic_bytes: {json.dumps(traffic, sort_keys=True)} -->")
    P("""
## SQ counters per dispatch (sums over the device)

MFMA busy fraction = SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs x kernel cycles), kernel cycles = SQ_BUSY_CYCLES / 32 shader
engines; clock = kernel cycles / average duration of the kernel-trace run. LDS active fraction =
SQ_LDS_IDX_ACTIVE / (256 CUs x kernel cycles). VALU per MFMA = (SQ_INSTS_VALU - SQ_INSTS_MFMA) / SQ_INSTS_MFMA.

| kernel | SQ_INSTS_MFMA | SQ_INSTS_VALU (incl. MFMA) | VALU per MFMA | MFMA busy cycles | MFMA+VALU co-exec cycles | LDS active cycles | LDS bank-conflict cycles | kernel cycles | clock GHz | MFMA busy fraction | LDS active fraction |
|---|---|---|---|---|---|---|---|---|---|---|---|""")
    for k in order:
        d = sq.get(k)
        if not d or not d.get("SQ_INSTS_MFMA"):
            continue
        cyc, ns = d["SQ_BUSY_CYCLES"] / 32, float(kt[k]["AverageNs"])
        P(f"| {k} | {d['SQ_INSTS_MFMA']:.0f} | {d['SQ_INSTS_VALU']:.0f} | {(d['SQ_INSTS_VALU'] - d['SQ_INSTS_MFMA']) / d['SQ_INSTS_MFMA']:.2f} | "
          f"{d['SQ_VALU_MFMA_BUSY_CYCLES']:.0f} | {d['SQ_VALU_MFMA_COEXEC_CYCLES']:.0f} | {d['SQ_LDS_IDX_ACTIVE']:.0f} | "
          f"{d['SQ_LDS_BANK_CONFLICT']:.0f} | {cyc:.0f} | {cyc / ns:.2f} | {d['SQ_VALU_MFMA_BUSY_CYCLES'] / 1024 / cyc:.3f} | "
          f"{d['SQ_LDS_IDX_ACTIVE'] / 256 / cyc:.3f} |")
    if args.note:
        P("\n" + args.note)


if __name__ == "__main__":
    main()
