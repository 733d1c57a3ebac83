"""Turns rocprofv3 CSV output into the short tables kept under profiles/.

    python -m axiom_amd.profile_summary trace   <dir>                  per-kernel launch counts and durations
    python -m axiom_amd.profile_summary counters <dir> [<dir> ...]     per-kernel averages of every collected counter
                                                                       (this library's kernels only)
    python -m axiom_amd.profile_summary traffic <FETCH_SIZE dir> <WRITE_SIZE dir>
                                                                       HBM bytes per launch of bench.py's workloads
    python -m axiom_amd.profile_summary survey  <bench.py output>      the `row_program_survey` of a bench line as a table
    python -m axiom_amd.profile_summary by-grid [--match=a,b] <dir> [<dir> ...]   durations and counter averages of the product kernels (or of those whose names contain a, b, ...)
                                                                       per (kernel, grid size): one kernel, several sizes

`<dir>` is what `rocprofv3 ... -f csv -d <dir> -o <name>` wrote: `<name>_kernel_trace.csv` and, for a counter run,
`<name>_counter_collection.csv` (searched recursively).  `traffic` scales FETCH_SIZE / WRITE_SIZE (KiB per dispatch) by
what the same counters read for bench.py's plain fp32 copy, whose traffic is known, and prints the table bench.py reads
its `traffic` fields from (first cell: the workload's key in backticks; last cell: bytes per launch).
"""
from __future__ import annotations

import collections
import csv
import sys
from pathlib import Path

# bench.py workload key -> (substring of the kernel name, algorithmic bytes per launch)
WORKLOADS = {
    "copy_f32_8192x8192": ("elementwise_kernel<256, 4>", 2 * 8192 * 8192 * 4),
    "chain_relu_add_mul_softmax_sum_f32_8192x8192": ("relu_adds_mulf_softmax_sum_f32", 2 * 8192 * 8192 * 4 + 8192 * 4),
    "chain_gelu_layernorm_bf16_16384x4096": ("layernorm_gelu_wb_bf16", 2 * 16384 * 4096 * 2 + 2 * 4096 * 2),
    "chain_gelu_rmsnorm_bf16_16384x4096": ("rmsnorm_gelu_w_bf16", 2 * 16384 * 4096 * 2 + 4096 * 2),
    "softmax_bf16_30000x1500_odd_row_length": ("axp_softmax_bf16_g64_it3_grid", 2 * 30000 * 1500 * 2),
    "sdpa_bf16_causal_b4h32s4096d128": ("sdpa_mfma_pingpong_kernel<true, 128>", 4 * 4 * 32 * 4096 * 128 * 2),
}
CALIBRATION = "copy_f32_8192x8192"


def _short(name: str) -> str:
    name = name.replace("(anonymous namespace)::", "").split("(")[0]
    return name if len(name) <= 96 else "..." + name[-93:]


def _find(d: str, suffix: str) -> list[Path]:
    return sorted(Path(d).rglob("*" + suffix))


def trace(d: str) -> None:
    dur = collections.defaultdict(list)
    for f in _find(d, "kernel_trace.csv"):
        for r in csv.DictReader(open(f)):
            dur[_short(r["Kernel_Name"])].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    print("| kernel | launches | average us | shortest us | share of kernel time |\n|---|---:|---:|---:|---:|")
    total = sum(sum(v) for v in dur.values())
    rest = 0.0
    for k, v in sorted(dur.items(), key=lambda kv: -sum(kv[1])):
        if sum(v) < 0.002 * total:  # input generation and checks by torch, runtime fills and copies
            rest += sum(v)
            continue
        print(f"| `{k}` | {len(v)} | {sum(v) / len(v):.1f} | {min(v):.1f} | {100 * sum(v) / total:.1f} % |")
    print(f"| (kernels under 0.2 % each) | | | | {100 * rest / total:.1f} % |")


def _counter_averages(d: str) -> dict:
    acc = collections.defaultdict(list)
    for f in _find(d, "counter_collection.csv"):
        for r in csv.DictReader(open(f)):
            acc[(_short(r["Kernel_Name"]), r["Counter_Name"])].append(float(r["Counter_Value"]))
    return {k: (sum(v) / len(v), len(v)) for k, v in acc.items()}


def counters(dirs: list[str]) -> None:
    table = collections.defaultdict(dict)
    for d in dirs:
        for (kernel, counter), (avg, n) in _counter_averages(d).items():
            table[kernel][counter] = avg
            table[kernel]["dispatches"] = n
    names = sorted({c for row in table.values() for c in row} - {"dispatches"})
    print("| kernel | dispatches | " + " | ".join(names) + " |\n|---|---:|" + "---:|" * len(names))
    for kernel, row in sorted(table.items()):
        if "axp_" not in kernel and "axhip::" not in kernel:
            continue
        print(f"| `{kernel}` | {row['dispatches']} | " + " | ".join(f"{row[c]:.4g}" if c in row else "" for c in names) + " |")


def traffic(fetch_dir: str, write_dir: str) -> None:
    fetch, write = _counter_averages(fetch_dir), _counter_averages(write_dir)

    def reading(table, counter, needle):
        hits = [(k, v) for (k, c), v in table.items() if c == counter and needle in k]
        return (hits[0][0], hits[0][1][0]) if hits else (None, None)

    _, cal_f = reading(fetch, "FETCH_SIZE", WORKLOADS[CALIBRATION][0])
    _, cal_w = reading(write, "WRITE_SIZE", WORKLOADS[CALIBRATION][0])
    if cal_f is None or cal_w is None:
        sys.exit("the calibration kernel (bench.py's plain fp32 copy) is not in these runs")
    known_kib = WORKLOADS[CALIBRATION][1] / 2 / 1024
    kf, kw = cal_f / known_kib, cal_w / known_kib
    print(f"Calibration on the plain fp32 copy ({known_kib:.0f} KiB read, {known_kib:.0f} KiB written): FETCH_SIZE reads {cal_f:.0f} KiB "
          f"(factor {kf:.5f}), WRITE_SIZE reads {cal_w:.0f} KiB (factor {kw:.5f}).\n")
    print("| workload | kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | read MB | written MB | algorithmic MB | traffic / algorithmic | HBM bytes per launch |")
    print("|---|---|---:|---:|---:|---:|---:|---:|---:|")
    for key, (needle, algo) in WORKLOADS.items():
        kn, f = reading(fetch, "FETCH_SIZE", needle)
        _, w = reading(write, "WRITE_SIZE", needle)
        if f is None or w is None:
            continue
        rd, wr = f / kf * 1024, w / kw * 1024
        print(f"| `{key}` | `{kn}` | {f:.0f} | {w:.0f} | {rd / 1e6:.1f} | {wr / 1e6:.1f} | {algo / 1e6:.1f} | {(rd + wr) / algo:.3f} | {rd + wr:.0f} |")


def survey(path: str) -> None:
    import json

    line = json.loads(Path(path).read_text().strip().splitlines()[-1])
    rows = line["row_program_survey"]
    print("| program | kernel | MB | us back to back | of HBM peak | us cold | cold, of HBM peak |\n|---|---|---:|---:|---:|---:|---:|")
    for name, r in rows.items():
        cold = f"{r['cold_us']:.1f} | {100 * r['frac_of_hbm_peak_cold']:.1f} %" if "cold_us" in r else " | "
        print(f"| `{name}` | `{r['kernel']}` | {r['bytes'] / 1e6:.0f} | {r['avg_us']:.1f} | {100 * r['frac_of_hbm_peak']:.1f} % | {cold} |")
    fr = [r["frac_of_hbm_peak"] for r in rows.values()]
    print(f"\nBack to back: {sum(f >= 0.7 for f in fr)} of {len(fr)} programs are at or above 70 % of the peak (lowest {100 * min(fr):.1f} %, highest {100 * max(fr):.1f} %); "
          f"every result finite: {all(r['finite'] for r in rows.values())}.")
    fc = [r["frac_of_hbm_peak_cold"] for r in rows.values() if "frac_of_hbm_peak_cold" in r]
    if fc:
        ov = sorted(r["event_overhead_us"] for r in rows.values() if "event_overhead_us" in r)
        print(f"Cold: {sum(f >= 0.7 for f in fc)} of {len(fc)} at or above 70 %, {sum(f >= 0.6 for f in fc)} at or above 60 % (lowest {100 * min(fc):.1f} %, highest "
              f"{100 * max(fc):.1f} %); the event bracketing that was taken off: median {ov[len(ov) // 2]:.1f} us per launch.")


def by_grid(dirs: list[str], needles: tuple[str, ...] = ("gemm", "Cijk")) -> None:
    """Durations and counter averages per (kernel, grid size): one kernel serves several problem sizes in a run.  A
    kernel whose grid is the same for every size (the vendor's stream-K kernels) is split at 130 us instead."""
    import collections
    import csv

    def short(n: str) -> str:
        n = n.replace("(axhip::GemmArgs, int, int)", "").split("(")[0]
        return n if len(n) < 70 else "..." + n[-60:]

    for d in dirs:
        dur = {}
        for f in _find(d, "kernel_trace.csv"):
            acc = collections.defaultdict(list)
            for r in csv.DictReader(open(f)):
                us = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
                dur[r["Dispatch_Id"]] = us
                if not any(n in r["Kernel_Name"] for n in needles):
                    continue
                grid = r.get("Grid_Size") or r.get("Grid_Size_X")
                if "MT256x256x64" in r["Kernel_Name"]:
                    grid += " short" if us < 130 else " long"
                acc[(short(r["Kernel_Name"]), grid)].append(us)
            for k, v in sorted(acc.items()):
                v.sort()
                print(f"{d}: `{k[0]}` grid {k[1]}: {len(v)} launches, average {sum(v) / len(v):.1f} us, median {v[len(v) // 2]:.1f}, shortest {v[0]:.1f}")
        for f in _find(d, "counter_collection.csv"):
            acc = collections.defaultdict(lambda: collections.defaultdict(list))
            for r in csv.DictReader(open(f)):
                if not any(n in r["Kernel_Name"] for n in needles):
                    continue
                grid = r.get("Grid_Size") or r.get("Grid_Size_X")
                if "MT256x256x64" in r["Kernel_Name"]:
                    grid += " short" if dur.get(r["Dispatch_Id"], 0) < 130 else " long"
                acc[(short(r["Kernel_Name"]), grid)][r["Counter_Name"]].append(float(r["Counter_Value"]))
            for k, cs in sorted(acc.items()):
                print(f"{d}: `{k[0]}` grid {k[1]}: " + " ".join(f"{c}={sum(v) / len(v):.4g}" for c, v in sorted(cs.items())))


def main() -> int:
    if len(sys.argv) >= 3 and sys.argv[1] == "trace":
        trace(sys.argv[2])
    elif len(sys.argv) >= 3 and sys.argv[1] == "counters":
        counters(sys.argv[2:])
    elif len(sys.argv) == 4 and sys.argv[1] == "traffic":
        traffic(sys.argv[2], sys.argv[3])
    elif len(sys.argv) >= 3 and sys.argv[1] == "by-grid":
        args = sys.argv[2:]
        if args[0].startswith("--match="):  # substrings of the kernel names to keep (default: the product kernels)
            by_grid(args[1:], tuple(args[0][len("--match="):].split(",")))
        else:
            by_grid(args)
    elif len(sys.argv) == 3 and sys.argv[1] == "survey":
        survey(sys.argv[2])
    else:
        print(__doc__, file=sys.stderr)
        return 2
    return 0


if __name__ == "__main__":
    sys.exit(main())
