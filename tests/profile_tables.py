"""The tables under profiles/ that bench.py reads and writes.

profiles/hbm_traffic.md holds the HBM-side bytes per launch of the headline kernels (`roofline.traffic` in the
benchmark line); profiles/bench_all_kernels_kernel_trace.md the per-kernel durations of a `rocprofv3
--kernel-trace --stats` run of the benchmark beside the benchmark's own event timing; profiles/kernel_counters.md
the hardware counters of the same kernels beside the vendor libraries' kernels and plain streaming kernels of the
same run; profiles/eval_sweeps.md the reference harnesses' sweeps. All are written from raw output files by the
functions below (`python bench.py --traffic-summary | --trace-summary | --counter-summary | --eval-summary DIR`),
never by hand, and tests/test_bench_tables.py checks that the traffic rows belong to the kernel sources in the
tree. No GPU work happens here.
"""
from __future__ import annotations

import hashlib
import json
import os
import re
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]
TRAFFIC_FILE = ROOT / "profiles" / "hbm_traffic.md"
KERNEL_SOURCE = {"sgemm": "sgemm.hip", "scan": "scan.hip", "gemm_bf16": "gemm_bf16.hip", "add_m": "add_m.hip"}


def source_hash(workload: str) -> str:
    """First 16 hex digits of the SHA-256 of the kernel source a workload runs."""
    return hashlib.sha256((ROOT / "prism_amd" / "csrc" / KERNEL_SOURCE[workload]).read_bytes()).hexdigest()[:16]


def measured_traffic(workload: str, size: int):
    """HBM-side bytes per launch (L2 misses: TCC fetches + write-backs) from profiles/hbm_traffic.md, the
    summary of two `rocprofv3 --pmc` runs of bench.py (FETCH_SIZE, then WRITE_SIZE, scaled by what the same
    counters read for a copy of known size). Each row records the hash of the kernel source it was measured
    on; a row whose hash differs from the source now in the tree is stale and gives None."""
    try:
        text = TRAFFIC_FILE.read_text()
    except OSError:
        return None
    for m in re.finditer(r"^\|\s*(\w+)\s*\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*([0-9a-f]{16})\s*\|", text, re.M):
        if m.group(1) == workload and int(m.group(2)) == size:
            return int(m.group(3)) + int(m.group(4)) if m.group(5) == source_hash(workload) else None
    return None


# ------------------------------------------------- HBM-side traffic table --

TRAFFIC_KERNELS = [  # (workload, size, substring of the kernel name, threads in the grid)
    ("sgemm", 8192, "sgemm_wave_tile_dma_kernel", 1024 * 1024),
    ("scan", 1 << 30, "scan_lookback_kernel", (1 << 30) // 65536 * 1024),
    ("gemm_bf16", 8192, "gemm_bf16_early_kernel<256, 256, 128, 128, false, float", 256 * 256),  # fp32 output; one workgroup per CU walks four tiles
    ("add_m", 1 << 24, "add_m_vec4_kernel", (1 << 24) // 4),
    ("add_m", 1 << 28, "add_m_vec4_kernel", (1 << 28) // 4),
]


def write_traffic_table(pmc_dir: str) -> int:
    """Summarises four `rocprofv3 --pmc` runs of bench.py into profiles/hbm_traffic.md, the table
    measured_traffic() reads. Expected in pmc_dir (rocprofv3 -d pmc_dir -o NAME --output-format csv):
    bench_FETCH_SIZE, bench_WRITE_SIZE (`bench.py --no-configs --no-cpu-baseline --steps 3 --warmup 1`) and
    calib_FETCH_SIZE, calib_WRITE_SIZE (`bench.py --workload calibrate --steps 3 --warmup 1`)."""
    import csv

    def readings(name, counter, match, grid=None):
        vals = []
        with open(os.path.join(pmc_dir, f"{name}_{counter}_counter_collection.csv"), newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] == counter and match in r["Kernel_Name"] and (grid is None or int(r["Grid_Size"]) == grid):
                    vals.append(float(r["Counter_Value"]))
        return vals

    scale = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        v = readings("calib", counter, "calibrate_copy_packet_kernel", (1 << 30) // 16)
        if not v:
            print(f"no copy kernel in calib_{counter}", file=sys.stderr)
            return 1
        scale[counter] = (1 << 20) / (sum(v) / len(v))  # the copy moves 1 GiB = 2^20 KiB each way
    lines = ["# HBM-side traffic per launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)", "",
             "Written by `python bench.py --traffic-summary $OUT/pmc_traffic` from four counter runs (from /tmp with TMPDIR=/tmp on",
             "the GPU box, R = repo root, OUT = a scratch directory, C = FETCH_SIZE, then WRITE_SIZE; each run its own process):", "",
             "    rocprofv3 --pmc $C --kernel-trace -d $OUT/pmc_traffic -o bench_$C --output-format csv -- \\",
             "        python3 $R/bench.py --steps 3 --warmup 1 --no-configs --no-cpu-baseline",
             "    rocprofv3 --pmc $C --kernel-trace -d $OUT/pmc_traffic -o calib_$C --output-format csv -- \\",
             "        python3 $R/bench.py --workload calibrate --steps 3 --warmup 1", "",
             "`bench.py` reads the table back for `roofline.traffic`. A row counts only while the hash of its kernel source",
             "(first 16 hex digits of the SHA-256 of `prism_amd/csrc/<file>`) is the one in the tree; otherwise the bench line",
             "says `null`. The counters sit at the L2's memory side, so they include what the 256 MiB memory-side cache serves.",
             "", f"Scale factors from the 1 GiB copy (calibrate_copy_packet_kernel): FETCH_SIZE x {scale['FETCH_SIZE']:.3f}, WRITE_SIZE x {scale['WRITE_SIZE']:.3f}"
             " (KiB per dispatch -> KiB moved).", "",
             "| workload | size | bytes read | bytes written | source hash | launches averaged | algorithmic bytes | ratio |",
             "|---|---:|---:|---:|---|---:|---:|---:|"]
    algorithmic = {("sgemm", 8192): 4 * 4 * 8192 ** 2, ("scan", 1 << 30): 8 << 30, ("gemm_bf16", 8192): (2 * 2 + 4) * 8192 ** 2,
                   ("add_m", 1 << 24): 8 << 24, ("add_m", 1 << 28): 8 << 28}
    for workload, size, match, grid in TRAFFIC_KERNELS:
        f, w = readings("bench", "FETCH_SIZE", match, grid), readings("bench", "WRITE_SIZE", match, grid)
        if not f or not w:
            print(f"no readings for {workload} {size}", file=sys.stderr)
            continue
        rd = int(sum(f) / len(f) * scale["FETCH_SIZE"] * 1024)
        wr = int(sum(w) / len(w) * scale["WRITE_SIZE"] * 1024)
        alg = algorithmic[(workload, size)]
        lines.append(f"| {workload} | {size} | {rd} | {wr} | {source_hash(workload)} | {min(len(f), len(w))} | {alg} | {(rd + wr) / alg:.3f} |")
    lines += ["", "The streaming kernels move their algorithmic bytes and nothing else (the scan's status words and polls are",
              "0.1 %). The GEMMs are compute-bound; their HBM-side reads are L2 misses of re-used A / B panels: with 256 x 256",
              "tiles and an 8 x 4 tile patch per XCD, 12 of the 64 panel reads of a patch miss, which is what an XCD's 32 CUs",
              "working in step can reach at best with that patch shape."]
    TRAFFIC_FILE.write_text("\n".join(lines) + "\n")
    print("\n".join(lines))
    return 0


# ------------------------------------------------------ kernel-trace table --

TRACE_FILE = ROOT / "profiles" / "bench_all_kernels_kernel_trace.md"
PEAKS = {"sgemm": (157.3, "TFLOP/s fp32 MFMA"), "gemm_bf16": (2500.0, "TFLOP/s bf16 MFMA"),
         "gemm_bf16_runmyh100": (2500.0, "TFLOP/s bf16 MFMA"), "scan": (8000.0, "GB/s HBM"),
         "scan_ticket_order": (8000.0, "GB/s HBM"), "add_m": (8000.0, "GB/s HBM"), "add_m_2p28": (8000.0, "GB/s HBM")}
TRACE_KERNELS = [  # (key of the benchmark line, substring of the kernel name, work per launch, unit divisor)
    ("sgemm", "sgemm_wave_tile_dma_kernel<256, 256, 32, 32, 128, false, false, false>", 2.0 * 8192 ** 3, 1e12),
    ("scan", "scan_lookback_kernel<prism::(anonymous namespace)::BigCfg, true, false, false", 8.0 * (1 << 30), 1e9),
    ("scan_ticket_order", "scan_lookback_kernel<prism::(anonymous namespace)::BigCfg, true, true, false", 8.0 * (1 << 30), 1e9),
    ("gemm_bf16", "gemm_bf16_early_kernel<256, 256, 128, 128, false, float", 2.0 * 8192 ** 3, 1e12),
    ("gemm_bf16_runmyh100", "gemm_bf16_early_kernel<256, 256, 128, 128, false, unsigned short", 2.0 * 8192 ** 3, 1e12),
    ("add_m_2p28", "add_m_vec4_kernel<true>", 8.0 * (1 << 28), 1e9),
    ("add_m", "add_m_vec4_kernel<false>", 8.0 * (1 << 24), 1e9),
]


def write_kernel_trace_table(prof_dir: str) -> int:
    """Summarises one `rocprofv3 --kernel-trace --stats` run of bench.py into
    profiles/bench_all_kernels_kernel_trace.md. Expected in prof_dir: bench_kernel_stats.csv (rocprofv3 -d prof_dir
    -o bench --output-format csv) and bench.json, the line the profiled run printed."""
    import csv

    with open(os.path.join(prof_dir, "bench_kernel_stats.csv"), newline="") as f:
        stats = list(csv.DictReader(f))
    with open(os.path.join(prof_dir, "bench.json")) as f:
        line = json.loads([l for l in f.read().splitlines() if l.startswith("{")][-1])
    timed = {"sgemm": line, **{k: v for k, v in line["also"].items() if isinstance(v, dict) and "ms" in v}}
    out = ["# rocprofv3 kernel-trace summary: bench.py, the headline workloads (MI355X, gfx950)", "",
           "Written by `python bench.py --trace-summary $OUT/prof_trace` from one profiled run (from /tmp with TMPDIR=/tmp on",
           "the GPU box, R = repo root, OUT = a scratch directory):", "",
           "    rocprofv3 --kernel-trace --stats -d $OUT/prof_trace -o bench --output-format csv -- \\",
           "        python3 $R/bench.py --no-configs --no-cpu-baseline > $OUT/prof_trace/bench.json", "",
           "Workloads: sgemm 8192^3 (kernel 5, alpha 1, beta 0.5), scan int32 n=2^30 (tiles by workgroup id, and by ticket), gemm_bf16 8192^3 (fp32 output, and",
           "the reference harness's entry with bf16 column-major output), add_m n=2^24 and 2^28.",
           f"Each kernel runs once for the parity gate, for {line.get('settle_ms', 150):.0f} ms of untimed settling, {line['warmup']} warm-up and {line['steps']} timed steps,",
           "hence the call counts; the profiler's average covers all of them (the cold first call is the `max` column), the",
           "last column is the benchmark's own event timing of the timed steps of the same run.", "",
           "| kernel (prism::) | calls | avg us | min us | max us | bench.py ms/step | achieved | peak | fraction |",
           "|---|---:|---:|---:|---:|---:|---:|---|---:|"]
    for key, match, work, div in TRACE_KERNELS:
        rows = [r for r in stats if match in r["Name"]]
        if not rows or key not in timed:
            print(f"no kernel or no timing for {key}", file=sys.stderr)
            continue
        r = max(rows, key=lambda r: float(r["TotalDurationNs"]))
        name = re.sub(r"^void ", "", r["Name"]).replace("prism::(anonymous namespace)::", "")
        name = name[: name.index("(")] if "(" in name else name
        ms = timed[key]["ms_per_step"] if key == "sgemm" else timed[key]["ms"]
        achieved = work / (ms * 1e-3) / div
        peak, unit = PEAKS[key]
        out.append(f"| `{name}` | {r['Calls']} | {float(r['AverageNs']) / 1e3:.2f} | {float(r['MinNs']) / 1e3:.2f} | "
                   f"{float(r['MaxNs']) / 1e3:.2f} | {ms:.4f} | {achieved:.1f} | {peak:g} {unit} | {achieved / peak:.3f} |")
    out += ["", "Work per launch: sgemm and gemm_bf16 2 * 8192^3 flop, scan 2 * 4 * 2^30 B, add_m 8 B per element. add_m at 2^24",
            "re-reads and re-writes the same 128 MiB every step, which the 256 MiB memory-side cache partly serves: the",
            "HBM-bound add_m figure is the 2^28 one.", "",
            "All kernels of this library in the run (the streaming calibration copies and PyTorch's own kernels left out):", "",
            "| kernel | calls | average us | total ms |", "|---|---:|---:|---:|"]
    for r in sorted(stats, key=lambda r: -float(r["TotalDurationNs"])):
        if "prism::" not in r["Name"]:
            continue
        name = re.sub(r"^void ", "", r["Name"]).replace("prism::(anonymous namespace)::", "")
        name = name[: name.index("(")] if "(" in name else name
        out.append(f"| `{name}` | {r['Calls']} | {float(r['AverageNs']) / 1e3:.1f} | {float(r['TotalDurationNs']) / 1e6:.1f} |")
    configs = os.path.join(prof_dir, "configs_kernel_stats.csv")
    if os.path.exists(configs):
        with open(configs, newline="") as f:
            stats = list(csv.DictReader(f))
        out += ["", "## The default run, configuration table included", "",
                "    rocprofv3 --kernel-trace --stats -d $OUT/prof_trace -o configs --output-format csv -- \\",
                "        python3 $R/bench.py --no-cpu-baseline", "",
                "`also.configs` adds SGEMM kernels 1, 2, 3, 6, 4, 5 at 1024^3 .. 8192^3, kernel 5 at the tail shapes (with and",
                "without a workspace where one is used), the scans of 2^20, 2^24 and 2^28 elements and the bf16 product at 4096^3 and",
                "16384^3. This table names the kernel each of them lands on; averages mix the sizes a kernel was launched at.", "",
                "| kernel | calls | average us | total ms |", "|---|---:|---:|---:|"]
        for r in sorted(stats, key=lambda r: -float(r["TotalDurationNs"])):
            if "prism::" not in r["Name"]:
                continue
            name = re.sub(r"^void ", "", r["Name"]).replace("prism::(anonymous namespace)::", "")
            name = name[: name.index("(")] if "(" in name else name
            out.append(f"| `{name}` | {r['Calls']} | {float(r['AverageNs']) / 1e3:.1f} | {float(r['TotalDurationNs']) / 1e6:.1f} |")
    TRACE_FILE.write_text("\n".join(out) + "\n")
    print("\n".join(out))
    return 0


# ------------------------------------------------ hardware counter tables --

COUNTER_FILE = ROOT / "profiles" / "kernel_counters.md"
COUNTER_PASSES = {
    "p1": "SQ_BUSY_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_INSTS_LDS SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT SQ_WAIT_INST_ANY",
    "p2": "GRBM_GUI_ACTIVE TCC_HIT_sum TCC_MISS_sum TCP_PENDING_STALL_CYCLES_sum",
    "p3": "SQ_WAVES SQ_WAVE_CYCLES SQ_WAIT_ANY SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR SQ_INSTS_SALU SQ_ACTIVE_INST_ANY GRBM_GUI_ACTIVE",
}
GEMM_ROWS = [  # (label, substrings that must all occur in the kernel name, grid size in threads)
    ("ours, SGEMM kernel 5 (fp32)", ["sgemm_wave_tile_dma_kernel<256, 256, 32, 32, 128, false, false, false>"], 1024 * 1024),
    ("rocBLAS `rocblas_sgemm` (fp32)", ["Cijk_Ailk_Bljk_SB_"], None),
    ("ours, bf16 in, fp32 out", ["gemm_bf16_early_kernel<256, 256, 128, 128, false, float"], 256 * 256),
    ("hipBLASLt, bf16 in, fp32 out", ["Cijk_Alik_Bljk_BSS_BH"], None),
    ("ours, bf16 in, bf16 column-major out", ["gemm_bf16_early_kernel<256, 256, 128, 128, false, unsigned short"], 256 * 256),
    ("hipBLASLt, bf16 in, bf16 column-major out", ["Cijk_Alik_Bljk_BBS_BH"], None),
]
STREAM_ROWS = [
    ("ours, scan 2^30 (tiles by workgroup id)", ["scan_lookback_kernel<", "BigCfg, true, false, false"], (1 << 30) // 64),
    ("ours, scan 2^30 (ticket order)", ["scan_lookback_kernel<", "BigCfg, true, true, false"], (1 << 30) // 64),
    ("hipCUB `DeviceScan::InclusiveSum` 2^30 (its scan kernel)", ["rocprim", "trampoline_kernel"], None),
    ("copy 2^30 x 4 B, the scan's tile shape", ["calibrate_copy_tile_kernel"], (1 << 30) // 64),
    ("copy 2^30 x 4 B, one packet per lane", ["calibrate_copy_packet_kernel"], (1 << 30) // 4),
    ("read only, 4 GiB", ["calibrate_read_kernel"], None),
    ("write only, 4 GiB", ["calibrate_write_kernel"], None),
    ("ours, add_m 2^28", ["add_m_vec4_kernel<true>"], (1 << 28) // 4),
]


def write_counter_table(pmc_dir: str) -> int:
    """Summarises three `rocprofv3 --pmc` runs of bench.py (COUNTER_PASSES, outputs p1, p2, p3 in pmc_dir) into
    profiles/kernel_counters.md: per kernel the mean over its dispatches of every counter, and what follows
    from them (clock, matrix-pipe duty, L2 hit rate, waves resident, share of cycles the vector L1 waits)."""
    import csv
    from collections import defaultdict

    def load(name):
        per = defaultdict(lambda: defaultdict(list))  # (kernel name, grid) -> counter -> values
        dur = defaultdict(dict)                       # (kernel name, grid) -> dispatch id -> ns
        path = os.path.join(pmc_dir, f"{name}_counter_collection.csv")
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                key = (r["Kernel_Name"], int(r["Grid_Size"]))
                per[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
                dur[key][r["Dispatch_Id"]] = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        return per, dur

    try:
        passes = {name: load(name) for name in COUNTER_PASSES}
    except OSError as e:
        print(f"{e}", file=sys.stderr)
        return 1

    def row_values(match, grid):
        """Counter means of the kernel (the one with most dispatches among those that match), from all passes."""
        vals, n, us = {}, 0, 0.0
        for name, (per, dur) in passes.items():
            keys = [k for k in per if all(m in k[0] for m in match) and (grid is None or k[1] == grid)]
            if not keys:
                continue
            k = max(keys, key=lambda k: len(dur[k]))
            d = sorted(dur[k].values())
            d = d[: max(1, len(d) * 9 // 10)]  # the cold first dispatches out
            if name == "p2":
                n, us = len(dur[k]), sum(d) / len(d) / 1e3
                vals["_name"], vals["_grid"] = k
            for c, v in per[k].items():
                vals.setdefault(f"{name}:{c}", sum(v) / len(v))
                vals.setdefault(c, sum(v) / len(v))
        return vals, n, us

    def short(name):
        name = re.sub(r"^void ", "", name).replace("prism::(anonymous namespace)::", "").replace("(anonymous namespace)::", "")
        name = name[: name.index("(")] if "(" in name else name
        return name if len(name) <= 72 else name[:69] + "..."

    out = ["# rocprofv3 --pmc: hardware counters of the headline kernels beside the vendor libraries' and plain streaming kernels", "",
           "Written by `python bench.py --counter-summary $OUT/pmc_counters` from three counter runs of the same program (from /tmp",
           "with TMPDIR=/tmp on the GPU box, R = repo root, OUT = a scratch directory; each pass its own process, because one pass",
           "holds at most 8 SQ, 4 TCC and 2 GRBM counters):", ""]
    for name, counters in COUNTER_PASSES.items():
        out += [f"    rocprofv3 --pmc {counters} \\",
                f"        --kernel-trace -d $OUT/pmc_counters -o {name} --output-format csv -- python3 $R/bench.py --steps 5 --warmup 1 --no-configs --no-cpu-baseline"]
    out += ["", "`bench.py` runs, in one process, our kernels at the headline sizes (8192^3, 2^30, 2^28), the vendor libraries called directly",
            "on the same operands (rocblas_sgemm, hipBLASLt matmul, hipcub::DeviceScan::InclusiveSum) and the plain streaming kernels of",
            "tests/native/calibrate_stream.hip on 4 GiB buffers. Every figure is the mean over a kernel's dispatches in the run; counters",
            "are sums over the 8 XCDs. Derived: shader cycles = GRBM_GUI_ACTIVE / 8; clock = cycles / duration (both of pass p2);",
            "matrix-pipe duty = SQ_VALU_MFMA_BUSY_CYCLES (p1) / 1024 SIMDs / cycles; L2 hit rate = TCC_HIT / (TCC_HIT + TCC_MISS);",
            "waves resident = 4 x SQ_WAVE_CYCLES / cycles (p3, cycles of p3); vector L1 waiting = TCP_PENDING_STALL_CYCLES / 256 CUs / cycles.",
            "Durations under counter collection are a few per cent above the untraced ones.", "",
            "## GEMM kernels at 8192^3", "",
            "| kernel | dispatches | duration us | clock GHz | matrix-pipe duty | duty x clock / 2.4 GHz | SQ_INSTS_VALU | SQ_INSTS_LDS | SQ_ACTIVE_INST_LDS | LDS bank conflict cycles | SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES | L2 hit |",
            "|---|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|"]
    names = []
    for label, match, grid in GEMM_ROWS:
        v, n, us = row_values(match, grid)
        if not n or "GRBM_GUI_ACTIVE" not in v:
            print(f"no dispatches for {label}", file=sys.stderr)
            continue
        cycles = v["p2:GRBM_GUI_ACTIVE"] / 8
        clock = cycles / (us * 1e3)
        duty = v.get("SQ_VALU_MFMA_BUSY_CYCLES", 0) / 1024 / cycles
        hit = v.get("TCC_HIT_sum", 0) / max(1.0, v.get("TCC_HIT_sum", 0) + v.get("TCC_MISS_sum", 0))
        names.append(f"* {label}: `{short(v['_name'])}`, {v['_grid'] // 256 if 'prism' not in v['_name'] else v['_grid']} "
                     + ("workgroups of 256 threads" if "prism" not in v["_name"] else "threads"))
        out.append(f"| {label} | {n} | {us:.1f} | {clock:.2f} | {duty:.3f} | {duty * clock / 2.4:.3f} | {v.get('SQ_INSTS_VALU', 0):.3g} | "
                   f"{v.get('SQ_INSTS_LDS', 0):.3g} | {v.get('SQ_ACTIVE_INST_LDS', 0):.3g} | {v.get('SQ_LDS_BANK_CONFLICT', 0):.3g} | "
                   f"{v.get('SQ_WAIT_INST_ANY', 0) / max(1.0, v.get('p1:SQ_WAVE_CYCLES', 1)):.3f} | {hit:.2f} |")
    out += ["", "Kernel names:", ""] + names
    out += ["", "The fp32 kernels run near the nominal 2.4 GHz and their duty x clock is the fraction of the 157.3 TFLOP/s peak that bench.py",
            "reports. The bf16 kernels, ours and the library's alike, are power-limited: the clock column is what the part holds under",
            "them, and the published 2.5 PFLOP/s assumes 2.4 GHz.", "",
            "## Streaming kernels", "",
            "| kernel | dispatches | duration us | GB/s | fraction of 8 TB/s | waves launched | waves resident | SQ_WAIT_ANY / SQ_WAVE_CYCLES | SQ_ACTIVE_INST_ANY / SQ_WAVE_CYCLES | vector-memory reads | writes | vector L1 waiting | L2 hit |",
            "|---|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|---:|"]
    moved = {"scan": 8.0 * (1 << 30), "hipCUB": 8.0 * (1 << 30), "copy": 8.0 * (1 << 30), "read": 4.0 * (1 << 30), "write": 4.0 * (1 << 30), "add_m": 8.0 * (1 << 28)}
    for label, match, grid in STREAM_ROWS:
        v, n, us = row_values(match, grid)
        if not n or "p3:GRBM_GUI_ACTIVE" not in v:
            print(f"no dispatches for {label}", file=sys.stderr)
            continue
        nbytes = next(b for k, b in moved.items() if k in label)
        cycles2, cycles3 = v["p2:GRBM_GUI_ACTIVE"] / 8, v["p3:GRBM_GUI_ACTIVE"] / 8
        wc = max(1.0, v.get("p3:SQ_WAVE_CYCLES", 1))
        hit = v.get("TCC_HIT_sum", 0) / max(1.0, v.get("TCC_HIT_sum", 0) + v.get("TCC_MISS_sum", 0))
        out.append(f"| {label} | {n} | {us:.1f} | {nbytes / us / 1e3:.0f} | {nbytes / us / 1e3 / 8000:.3f} | {v.get('SQ_WAVES', 0):.0f} | "
                   f"{4 * wc / cycles3:.0f} | {v.get('SQ_WAIT_ANY', 0) / wc:.3f} | {v.get('SQ_ACTIVE_INST_ANY', 0) / wc:.3f} | "
                   f"{v.get('SQ_INSTS_VMEM_RD', 0):.0f} | {v.get('SQ_INSTS_VMEM_WR', 0):.0f} | "
                   f"{v.get('TCP_PENDING_STALL_CYCLES_sum', 0) / 256 / cycles2:.3f} | {hit:.2f} |")
    out += ["", "A scan tile of 65536 elements issues 16 x 16 data loads and as many stores; what the scan's vector-memory counts exceed",
            "the tile-shaped copy's by is its status traffic (header read, look-back polls, aggregate / prefix / cleared word). The scan",
            "stands beside the copy in its own tile shape, the copy with one packet per lane is the shape add_m uses, and the one-way",
            "streams show what the memory system gives in each direction."]
    COUNTER_FILE.write_text("\n".join(out) + "\n")
    print("\n".join(out))
    return 0


# ------------------------------------------- sweeps of the evaluation report --

def parse_eval_report(text: str):
    """The three sweeps of `python -m prism_amd.eval_report ...` (the reference harnesses' text formats) as
    ({size: {"vendor" | kernel number: GFLOPS}}, [(n, vendor GB/s, ours GB/s)], {size: {"Kernel" | "cuBLAS": TFLOPS}})."""
    sgemm, scan, h100 = {}, [], {}
    size = kernel = None
    in_table = False
    for line in text.splitlines():
        t = line.strip()
        m = re.match(r"Size:\s+(\d+)x\d+x\d+", t)
        if m:
            size = int(m.group(1))
        if t == "[cuBLAS FP32]":
            kernel = "vendor"
        m = re.match(r"\[My Kernel (\d+)\]", t)
        if m:
            kernel = int(m.group(1))
        m = re.search(r"performance:\s+\(\s*([\d.]+)\)\s+GFLOPS", t)
        if m and kernel is not None and size is not None:
            sgemm.setdefault(size, {})[kernel] = float(m.group(1))
            kernel = None
        m = re.match(r"(Kernel|cuBLAS):\s+.*performance:\s+\(\s*([\d.]+)\)\s+TFLOPS.*size:\s+\((\d+)\)", t)
        if m:
            h100.setdefault(int(m.group(3)), {})[m.group(1)] = float(m.group(2))
        if "Size" in t and "CUB (GB/s)" in t:
            in_table = True
            continue
        if in_table and t.startswith("---"):
            continue
        if in_table and t:
            parts = re.split(r"\s*\|\s*", t)
            scan.append((int(parts[0]), float(parts[1].split()[1]), float(parts[2].split()[1])))
        elif in_table:
            in_table = False
    return sgemm, scan, h100


def write_eval_tables(report_dir: str) -> int:
    """Summarises two runs of the evaluation sweeps into profiles/eval_sweeps.md. Expected in report_dir:
    eval_report.txt (`python -m prism_amd.eval_report`) and eval_generated.txt (`python -m prism_amd.eval_report
    generated`)."""
    out = ["# The reference harnesses' sweeps on one MI355X: hand-written kernels, DSL-generated kernels, vendor libraries", "",
           "Written by `python bench.py --eval-summary $OUT` from two runs on the GPU box (R = repo root, OUT = a scratch",
           "directory):", "",
           "    python3 -m prism_amd.eval_report > $OUT/eval_report.txt", "    python3 -m prism_amd.eval_report generated > $OUT/eval_generated.txt", "",
           "Protocols and text formats are the reference's (evals/4090_sgemm/main.cu:154-217: 10 launches between two events,",
           "alpha 0.5, beta 3.0; evals/4090_scan/bench.cu:157-262: best wall-clock of launch + sync; evals/h100_bench/main.cu:112-167:",
           "8 launches between two events). The vendor columns are rocblas_sgemm, hipcub::DeviceScan::InclusiveSum and a hipBLASLt",
           "bf16 matmul called directly (prism_amd/csrc/vendor/vendor_baselines.hip). The large GEMMs are timed right after the",
           "first call, while the clocks still settle, and read a few per cent below the sustained figures of bench.py.", ""]
    for name, title in (("eval_report.txt", "Hand-written kernels (libprism_amd.so)"), ("eval_generated.txt", "Kernels printed by the DSL back-end (prism_amd/examples)")):
        path = os.path.join(report_dir, name)
        if not os.path.exists(path):
            print(f"no {name} in {report_dir}", file=sys.stderr)
            continue
        sgemm, scan, h100 = parse_eval_report(open(path).read())
        out += [f"## {title}", ""]
        if sgemm:
            kernels = sorted({k for row in sgemm.values() for k in row if k != "vendor"})
            out += ["SGEMM, TFLOP/s (fraction of the 157.3 TFLOP/s fp32 MFMA peak for kernel 5):", "",
                    "| size | rocBLAS | " + " | ".join(f"kernel {k}" for k in kernels) + " |", "|---:|---:|" + "---:|" * len(kernels)]
            for size in sorted(sgemm):
                row = sgemm[size]
                cells = []
                for k in kernels:
                    v = row.get(k)
                    cells.append("-" if v is None else f"{v / 1e3:.1f}" + (f" ({v / 1e3 / 157.3:.2f})" if k == 5 else ""))
                out.append(f"| {size} | {row.get('vendor', 0) / 1e3:.1f} | " + " | ".join(cells) + " |")
            out.append("")
        if scan:
            out += ["Inclusive scan of uint32, GB/s (fraction of the 8 TB/s HBM peak):", "", "| n | hipCUB | ours |", "|---:|---:|---:|"]
            out += [f"| 2^{n.bit_length() - 1} | {v:.0f} | {o:.0f} ({o / 8000:.2f}) |" for n, v, o in scan]
            out.append("")
        if h100:
            out += ["bf16 GEMM, TFLOP/s (fraction of the 2.5 PFLOP/s bf16 MFMA peak):", "", "| size | hipBLASLt | ours |", "|---:|---:|---:|"]
            out += [f"| {n} | {r.get('cuBLAS', 0):.0f} | {r.get('Kernel', 0):.0f} ({r.get('Kernel', 0) / 2500:.2f}) |" for n, r in sorted(h100.items())]
            out.append("")
    (ROOT / "profiles" / "eval_sweeps.md").write_text("\n".join(out) + "\n")
    print("\n".join(out))
    return 0
