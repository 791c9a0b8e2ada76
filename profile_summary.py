"""Turns the raw rocprofv3 output of profile_counters.sh into the tables kept under profiles/.

    python profile_summary.py <output directory of profile_counters.sh> [commit]

Prints markdown, per workload of bench.py (`--profile-leg`): per-kernel durations from the kernel
trace, HBM bytes per launch from FETCH_SIZE / WRITE_SIZE (KiB per dispatch, each scaled by what the
same counter reads for the plain 1 GiB copy of `bench.py --copy-calibration`), the shader counters
per launch, and the lines that bench.py reads back for the `traffic` fields of its roofline objects:
`HBM_TRAFFIC <kernel> bytes_per_launch=<n> measured_at=<commit>` per library kernel of the headline
workload and `HBM_TRAFFIC_STEP <workload> bytes_per_step=<n> measured_at=<commit>` per workload.
"""
import csv
import os
import re
import subprocess
import sys
from collections import defaultdict

OURS = ("retention_", "suffix_intra", "short_seq", "segment_scan", "segment_contrib", "decode_step", "rotary_qk", "gated_norm")
COPY_KIB = 1 << 20   # the calibration copies 1 GiB


def short(name):
    name = re.sub(r"^void ", "", name).replace("(anonymous namespace)::", "")
    return re.sub(r"\(.*\)$", "", name)


def kernel_stats(path):
    rows = []
    with open(path) as f:
        for r in csv.DictReader(f):
            if any(k in r["Name"] for k in OURS):
                rows.append((short(r["Name"]), int(r["Calls"]), float(r["AverageNs"]) / 1e3, int(r["MinNs"]) / 1e3,
                             int(r["MaxNs"]) / 1e3))
    return sorted(rows, key=lambda r: -r[1] * r[2])


def counters(path):
    """-> {kernel: {counter: (mean value per dispatch, dispatches)}}"""
    acc = defaultdict(lambda: defaultdict(list))
    with open(path) as f:
        for r in csv.DictReader(f):
            acc[short(r["Kernel_Name"])][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return {k: {c: (sum(v) / len(v), len(v)) for c, v in cs.items()} for k, cs in acc.items()}


def copy_reading(path, counter):
    """The counter's largest per-dispatch value in the calibration run: the 1 GiB copy kernel."""
    best = 0.0
    for cs in counters(path).values():
        if counter in cs:
            best = max(best, cs[counter][0])
    return best


FAMILIES = (
    ("retention kernels of this library", ("retention_", "suffix_intra", "short_seq", "segment_scan", "segment_contrib", "decode_step")),
    ("rotary embedding kernel of this library", ("rotary_qk",)),
    ("norm + gate kernels of this library", ("gated_norm",)),
    ("GEMMs (rocBLAS / hipBLASLt)", ("Cijk_", "gemm", "Gemm")),
)


def model_breakdown(path):
    """Where the time of the traced run goes, by kernel family (the run holds bench.py's headline
    leg and its model leg; the headline leg's 12 forward + backward launches are a fraction of a
    per cent of it)."""
    rows = []
    with open(path) as f:
        for r in csv.DictReader(f):
            rows.append((r["Name"], int(r["Calls"]), int(r["TotalDurationNs"])))
    total = sum(r[2] for r in rows)
    print("\n## Model-level run (config 5 harness): GPU time by kernel family\n")
    print("| family | launches | total | share of GPU time |\n|---|---|---|---|")
    rest_calls, rest_ns = 0, 0
    fam = {name: [0, 0] for name, _ in FAMILIES}
    for name, calls, ns in rows:
        for fname, keys in FAMILIES:
            if any(k in name for k in keys):
                fam[fname][0] += calls
                fam[fname][1] += ns
                break
        else:
            rest_calls += calls
            rest_ns += ns
    for fname, _ in FAMILIES:
        print(f"| {fname} | {fam[fname][0]} | {fam[fname][1] / 1e6:.2f} ms | {100 * fam[fname][1] / total:.1f} % |")
    print(f"| everything else (torch elementwise, reductions, copies, losses) | {rest_calls} | {rest_ns / 1e6:.2f} ms | {100 * rest_ns / total:.1f} % |")
    print(f"| all kernels | {sum(r[1] for r in rows)} | {total / 1e6:.2f} ms | 100 % |")
    print("\nLibrary kernels in this run:\n\n| kernel | calls | average | total |\n|---|---|---|---|")
    for name, calls, ns in sorted(rows, key=lambda r: -r[2]):
        if any(k in name for k in OURS):
            print(f"| {short(name)} | {calls} | {ns / calls / 1e3:.1f} us | {ns / 1e6:.2f} ms |")


LEGS = (
    ("headline", "config 2: plain retention forward + backward (B8 H16 T4096 dk = dv = 128)"),
    ("pop_fused", "config 4 through flash_pop_retention_with_suffixes (config 2 + 65 suffixes x 16 tokens per sequence)"),
    ("pop_two_op", "config 4 through the reference's call sequence (flash_pop_retention, torch.cat, fused_chunk_retention)"),
    ("long", "config 3: B2 H8 T16384 dk128 dv256 with carried state (split-sequence entry points)"),
    ("layer5", "the retention op of one layer of config 5: fused POP step, B8 T2048 H12 dk64 dv128"),
    ("layer_ops", "the elementwise stages around the op at config 2's tensor shapes (B8 T4096 H16 d128): rotary, norm + gate forward and backward"),
)


def steps_of(log_path, default=8):
    """K of the `--profile-leg` run, from the JSON line it printed."""
    try:
        m = re.search(r'"steps": (\d+)', open(log_path).read())
        return int(m.group(1)) if m else default
    except OSError:
        return default


def main():
    out = sys.argv[1]
    commit = sys.argv[2] if len(sys.argv) > 2 else subprocess.run(
        ["git", "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip() or "unknown"
    p = lambda *a: os.path.join(out, *a)
    have_copy = os.path.exists(p("copy_fetch", "r_counter_collection.csv"))
    if have_copy:
        cf, cw = copy_reading(p("copy_fetch", "r_counter_collection.csv"), "FETCH_SIZE"), copy_reading(
            p("copy_write", "r_counter_collection.csv"), "WRITE_SIZE")
        sf, sw = COPY_KIB / cf, COPY_KIB / cw
        print(f"The 1 GiB copy kernel of `bench.py --copy-calibration` reads FETCH_SIZE = {cf:,.0f} KiB and WRITE_SIZE = {cw:,.0f} KiB "
              f"for a true 1 048 576 KiB each way: scale factors x {sf:.3f} and x {sw:.3f}.")
    machine = []
    for leg, what in LEGS:
        if not os.path.exists(p(f"trace_{leg}", "r_kernel_stats.csv")):
            continue
        print(f"\n# `--profile-leg {leg}` -- {what}\n")
        print("## Kernel trace (--kernel-trace --stats, after 0.3 s of the same steps)\n")
        print("| kernel | calls | average | min | max |\n|---|---|---|---|---|")
        for name, calls, avg, lo, hi in kernel_stats(p(f"trace_{leg}", "r_kernel_stats.csv")):
            print(f"| {name} | {calls} | {avg:.1f} us | {lo:.1f} us | {hi:.1f} us |")
        if have_copy and os.path.exists(p(f"fetch_{leg}", "r_counter_collection.csv")):
            fetch, write = counters(p(f"fetch_{leg}", "r_counter_collection.csv")), counters(p(f"write_{leg}", "r_counter_collection.csv"))
            k = steps_of(p(f"fetch_{leg}.log"))
            print(f"\n## HBM traffic ({k} steps, no spin-up; KiB per dispatch, scaled by the copy's factors)\n")
            print("| kernel | launches per step | FETCH_SIZE (KiB) | WRITE_SIZE (KiB) | read, scaled | written, scaled | total per launch |\n|---|---|---|---|---|---|---|")
            total = 0.0
            for name in sorted(fetch):
                if not any(o in name for o in OURS) or "FETCH_SIZE" not in fetch[name] or name not in write:
                    continue
                f_kib, n = fetch[name]["FETCH_SIZE"]
                w_kib = write[name]["WRITE_SIZE"][0]
                rd, wr = f_kib * sf * 1024, w_kib * sw * 1024
                total += (rd + wr) * n / k
                print(f"| {name} | {n / k:g} | {f_kib:,.0f} | {w_kib:,.0f} | {rd / 1e6:.1f} MB | {wr / 1e6:.1f} MB | {(rd + wr) / 1e6:.1f} MB |")
                if leg == "headline":
                    machine.append(f"HBM_TRAFFIC {name} bytes_per_launch={int(rd + wr)} measured_at={commit}")
            print(f"\nAll launches of the library in one step: {total / 1e6:.1f} MB.")
            machine.append(f"HBM_TRAFFIC_STEP {leg} bytes_per_step={int(total)} measured_at={commit}")
        for run in ("sq1", "sq2"):
            path = p(f"{run}_{leg}", "r_counter_collection.csv")
            if not os.path.exists(path):
                continue
            cs = counters(path)
            names = sorted(k for k in cs if any(o in k for o in ("retention_", "suffix_intra", "segment_contrib", "short_seq", "rotary_qk", "gated_norm")))
            ctrs = sorted({c for k in names for c in cs[k]})
            print(f"\n## Shader counters per launch ({run})\n")
            print("| counter | " + " | ".join(names) + " |\n|---|" + "---|" * len(names))
            for c in ctrs:
                print(f"| {c} | " + " | ".join(f"{cs[k][c][0]:,.0f}" if c in cs[k] else "" for k in names) + " |")
    if machine:
        print("\nRead back by bench.py (`roofline.traffic`):\n")
        for l in machine:
            print(l)
    if os.path.exists(p("trace_model", "r_kernel_stats.csv")):
        model_breakdown(p("trace_model", "r_kernel_stats.csv"))


if __name__ == "__main__":
    main()
