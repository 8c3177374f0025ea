#!/usr/bin/env python3
"""Profiles of bench.py under rocprofv3, turned into the short summaries kept under profiles/.

    python3 bench_profiles.py trace   --workload c3      # rocprofv3 --kernel-trace --stats of `bench.py --step-only`
    python3 bench_profiles.py traffic --workload c3      # two --pmc runs (FETCH_SIZE, then WRITE_SIZE) + copy calibration
    python3 bench_profiles.py counters --workload c3     # one --pmc run of SQ counters: MFMA and VALU busy, LDS, waits
    python3 bench_profiles.py issue --workload c3        # one --pmc run: matrix / vector co-execution, address unit queues
    python3 bench_profiles.py memsys --workload c3       # three --pmc runs: L2 hit rate, requests to memory, stalled channels
    python3 bench_profiles.py yardstick                  # no profiler: `bench.py --copy-yardstick` as a table

Each sub-command starts rocprofv3 as a child process with `python3 bench.py ...` after `--`, reads the CSV files it
leaves in a scratch directory (--raw-dir, default: a fresh temporary one), and prints a markdown summary (redirect it
into profiles/bench_<workload>_*.md).
`--step-only` makes bench.py launch nothing but the step and the kernels of the step, each op the same number of
times, so every kernel name in a trace is one op of one workload.

The traffic summary is what bench.py reads `roofline.traffic` from (column "traffic MB" of the row whose first
cell is the op's name in the bench line).
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.abspath(__file__))
OUT = None      # where rocprofv3 leaves its raw files: --raw-dir, or a temporary directory made on first use

# kernel name (substring) -> the op's key in the bench line; first match wins
KERNEL_KEYS = [
    ("row_gather_pair_kernel", "depad+transpose_pad_valid_rows"),
    ("DepadRowsMap", "depad"),
    ("DepadHeadsMap", "transpose_depad"),
    ("PadMap", "transpose_pad_valid_rows"),
    ("attn_qk", "attn_qk"),
    ("softmax", "scale_mask_softmax"),
    ("attn_pv", "attn_pv"),
    ("layernorm", "layernorm_residual"),
    ("decode_attn", "decode_attn"),
    ("decode_qk", "decode_qk"),
    ("decode_pv", "decode_pv"),
    ("attn_fused_wide", "attn_fused_packed_wide"),
    ("attn_fused", "attn_fused_packed"),
    ("copy_kernel", "copy"),
]

def key_of(kernel: str, decode: bool):
    for sub, key in KERNEL_KEYS:
        if sub in kernel:
            return key
    return None


def run_profiler(tag: str, prof_args, bench_args, timeout_s: int):
    """rocprofv3 <prof_args> -d <raw dir>/<tag> -- python3 bench.py <bench_args>; returns (dir, bench line, command)."""
    global OUT
    if OUT is None:
        OUT = tempfile.mkdtemp(prefix="energon_prof_")
    d = os.path.join(OUT, tag)
    subprocess.run(["rm", "-rf", d], check=True)
    os.makedirs(d, exist_ok=True)
    cmd = ["rocprofv3"] + prof_args + ["--output-format", "csv", "-d", d, "-o", "run", "--",
                                      "python3", os.path.join(ROOT, "bench.py")] + bench_args
    env = dict(os.environ, TMPDIR="/tmp")
    print("[bench_profiles] " + " ".join(cmd), file=sys.stderr, flush=True)
    proc = subprocess.run(cmd, cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                          timeout=timeout_s)
    if proc.returncode != 0:
        sys.stderr.write(proc.stderr[-3000:])
        raise SystemExit(f"rocprofv3 exited with {proc.returncode}")
    line = None
    for ln in proc.stdout.splitlines():
        if ln.startswith("{"):
            line = json.loads(ln)
    return d, line, " ".join(cmd[:1] + prof_args + ["--", "python3", "bench.py"] + bench_args)


def print_sources(line) -> None:
    """Names the library sources the profiled run was made on (en_source_hash, carried in the bench line):
    bench.py compares it with the library it runs before it takes a figure from the summary for that library's."""
    h = (line or {}).get("library_source_hash")
    if h is None:
        from energonai_amd import build
        h = build.source_hash()
    print(f"Library sources (`en_source_hash`) of the profiled run: `{h}`\n")


def find_csv(d: str, suffix: str) -> str:
    hits = glob.glob(os.path.join(d, "**", f"*{suffix}"), recursive=True)
    if not hits:
        raise SystemExit(f"no *{suffix} under {d}")
    return hits[0]


def trace_rows(path: str):
    agg = collections.defaultdict(list)
    with open(path) as f:
        for r in csv.DictReader(f):
            agg[r["Kernel_Name"]].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return agg


def counter_rows(path: str, counter: str):
    agg = collections.defaultdict(list)
    with open(path) as f:
        for r in csv.DictReader(f):
            if r["Counter_Name"] == counter:
                agg[r["Kernel_Name"]].append(float(r["Counter_Value"]))
    return agg


def cmd_trace(ns) -> int:
    bench_args = ["--workload", ns.workload, "--form", ns.form, "--step-only", "--no-cpu", "--steps", str(ns.steps),
                  "--warmup", str(ns.warmup)]
    d, line, shown = run_profiler(f"kt_{ns.workload}_{ns.form}", ["--kernel-trace", "--stats"], bench_args, ns.timeout)
    agg = trace_rows(find_csv(d, "kernel_trace.csv"))
    decode = ns.workload == "c5"
    kt = (line or {}).get("step_kernels", {})
    print(f"# rocprofv3 kernel-trace summary: `bench.py --workload {ns.workload} --form {ns.form} --step-only`\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout):\n")
    print(f"```\npython3 bench_profiles.py trace --workload {ns.workload} --form {ns.form}\n  -> {shown}\n```\n")
    print_sources(line)
    if line:
        print(f"Bench line of the profiled run: {line['ms_per_step'] * 1e3:.1f} us per step "
              f"({line['config']['workload']}). Event timings of the same run (`us (events)`) are taken by bench.py "
              f"with HIP events on the launch stream, back-to-back launches; the profiler's own durations are "
              f"per dispatch.\n")
    print("| op (key in the bench line) | kernel | calls | avg us | min us | max us | us (events) |\n|---|---|---|---|---|---|---|")
    for name, v in sorted(agg.items(), key=lambda kv: -sum(kv[1])):
        key = key_of(name, decode)
        if key is None:
            continue
        ev = kt.get(key, {}).get("us")
        print(f"| `{key}` | `{name[:100]}` | {len(v)} | {sum(v) / len(v):.1f} | {min(v):.1f} | {max(v):.1f} | "
              f"{'' if ev is None else format(ev, '.1f')} |")
    other = sum(sum(v) for n, v in agg.items() if key_of(n, decode) is None)
    print(f"\nOther kernels in the trace (torch fills and copies while the inputs are made): {other / 1e3:.1f} ms in total.")
    return 0


def cmd_traffic(ns) -> int:
    bench_args = ["--workload", ns.workload, "--form", ns.form, "--step-only", "--no-cpu", "--steps", str(ns.steps),
                  "--warmup", str(ns.warmup)]
    decode = ns.workload == "c5"
    per_counter, shown_cmds, line = {}, [], None
    calib = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        d, line, shown = run_profiler(f"pmc_{counter}_{ns.workload}_{ns.form}", ["--pmc", counter], bench_args, ns.timeout)
        shown_cmds.append(shown)
        per_counter[counter] = counter_rows(find_csv(d, "counter_collection.csv"), counter)
        d, cline, shown = run_profiler(f"pmc_{counter}_copy", ["--pmc", counter], ["--copy-yardstick", "--step-only", "--steps", "5"],
                                       ns.timeout)
        shown_cmds.append(shown)
        rows = counter_rows(find_csv(d, "counter_collection.csv"), counter)
        vals = [v for n, vs in rows.items() if "copy_kernel" in n for v in vs]
        # the copy kernel moves 64 MiB, 256 MiB and 1 GiB each way; the largest launches dominate the maximum
        calib[counter] = (1 << 30) / max(vals)      # bytes per counter unit
    alg = {k: v["alg_MB"] * 1e6 for k, v in (line or {}).get("step_kernels", {}).items()}
    # every op of the step is launched the same number of times in a --step-only run
    keys = collections.defaultdict(lambda: {"FETCH_SIZE": 0.0, "WRITE_SIZE": 0.0, "names": set(), "n": 0})
    for counter, rows in per_counter.items():
        for name, vals in rows.items():
            key = key_of(name, decode)
            if key is None or key == "copy":
                continue
            keys[key][counter] += sum(vals)
            keys[key]["names"].add(name[:70])
            keys[key]["n"] = max(keys[key]["n"], len(vals))
    calls = max((v["n"] for k, v in keys.items() if k == "layernorm_residual"), default=0) or \
        max(v["n"] for v in keys.values())
    print(f"# HBM traffic per launch, `bench.py --workload {ns.workload} --form {ns.form} --step-only`, from FETCH_SIZE / WRITE_SIZE\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout; one counter per run):\n")
    print(f"```\npython3 bench_profiles.py traffic --workload {ns.workload} --form {ns.form}")
    for c in shown_cmds:
        print(f"  -> {c}")
    print("```\n")
    print_sources(line)
    print(f"Calibration: the same counters over `en_copy_bytes` of 1 GiB (reads 1 GiB, writes 1 GiB) give "
          f"{calib['FETCH_SIZE']:.1f} bytes per FETCH_SIZE unit and {calib['WRITE_SIZE']:.1f} bytes per WRITE_SIZE unit; "
          f"the columns below are scaled by that. Each op ran {calls} times; traffic = counter total / {calls}.\n")
    print("| op (key in the bench line) | kernels | read MB | written MB | traffic MB | algorithmic MB | traffic / algorithmic |\n"
          "|---|---|---|---|---|---|---|")
    for key, v in keys.items():
        rd = v["FETCH_SIZE"] * calib["FETCH_SIZE"] / calls / 1e6
        wr = v["WRITE_SIZE"] * calib["WRITE_SIZE"] / calls / 1e6
        a = alg.get(key)
        if key == "depad+transpose_pad_valid_rows":
            a = alg.get("depad", 0) + alg.get("transpose_pad_valid_rows", 0)
        print(f"| `{key}` | {'; '.join(sorted(v['names']))} | {rd:.1f} | {wr:.1f} | {rd + wr:.1f} | "
              f"{'' if not a else format(a / 1e6, '.1f')} | {'' if not a else format((rd + wr) * 1e6 / a, '.2f')} |")
    print("\nReads below the algorithmic figure are hits in the 256 MB memory-side cache, which FETCH_SIZE does not count "
          "as HBM traffic; writes above it are whole 16-byte vectors at ragged row ends.")
    return 0


SQ_COUNTERS = ["SQ_WAVE_CYCLES", "SQ_VALU_MFMA_BUSY_CYCLES", "SQ_ACTIVE_INST_VALU", "SQ_LDS_BANK_CONFLICT",
               "SQ_LDS_IDX_ACTIVE", "SQ_WAIT_INST_ANY", "SQ_BUSY_CU_CYCLES", "GRBM_GUI_ACTIVE"]


def cmd_counters(ns) -> int:
    # --all-ops: the whole bench line of the workload instead of the step alone, so that the ops the step does not
    # launch (fused attention, the movers of the reference's sequence) are counted too; a kernel name then mixes
    # the forms that share it
    scope = ["--no-extra"] if ns.all_ops else ["--form", ns.form, "--step-only"]
    bench_args = ["--workload", ns.workload] + scope + ["--no-cpu", "--steps", str(ns.steps), "--warmup", str(ns.warmup)]
    decode = ns.workload == "c5"
    d, line, shown = run_profiler(f"sq_{ns.workload}", ["--pmc"] + SQ_COUNTERS, bench_args, ns.timeout)
    path = find_csv(d, "counter_collection.csv")
    per = {c: counter_rows(path, c) for c in SQ_COUNTERS}
    keys = collections.defaultdict(lambda: collections.defaultdict(float))
    names = collections.defaultdict(set)
    for c, rows in per.items():
        for name, vals in rows.items():
            key = key_of(name, decode)
            if key is None or key == "copy":
                continue
            keys[key][c] += sum(vals)
            keys[key]["n_" + c] += len(vals)
            names[key].add(name[:70])
    print(f"# SQ counters of the kernels of `bench.py --workload {ns.workload} {' '.join(scope)}`\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout):\n")
    print(f"```\npython3 bench_profiles.py counters --workload {ns.workload}"
          f"{' --all-ops' if ns.all_ops else ' --form ' + ns.form}\n  -> {shown}\n```\n")
    print_sources(line)
    print("All columns are sums over the launches of an op divided as stated.  `GRBM_GUI_ACTIVE` is summed over the 8 "
          "XCDs, so SIMD cycles of a launch = GRBM_GUI_ACTIVE / 8 x 1024 SIMDs.  `SQ_WAVE_CYCLES`, "
          "`SQ_ACTIVE_INST_VALU` and `SQ_WAIT_INST_ANY` count in units of four cycles.\n")
    print("| op (key in the bench line) | kernels | MFMA busy, share of SIMD cycles | VALU issue, share of SIMD cycles | "
          "resident waves per SIMD | waves waiting at s_waitcnt, share of wave time | CUs with a wave, of 256 | "
          "LDS bank conflict cycles / LDS active cycles |\n|---|---|---|---|---|---|---|---|")
    for key, v in keys.items():
        simd = v["GRBM_GUI_ACTIVE"] / 8 * 1024
        if simd <= 0:
            continue
        lds = v["SQ_LDS_IDX_ACTIVE"]
        print(f"| `{key}` | {'; '.join(sorted(names[key]))} | {v['SQ_VALU_MFMA_BUSY_CYCLES'] / simd:.3f} | "
              f"{4 * v['SQ_ACTIVE_INST_VALU'] / simd:.3f} | {4 * v['SQ_WAVE_CYCLES'] / simd:.2f} | "
              f"{v['SQ_WAIT_INST_ANY'] / max(v['SQ_WAVE_CYCLES'], 1):.3f} | "
              f"{v['SQ_BUSY_CU_CYCLES'] / (v['GRBM_GUI_ACTIVE'] / 8):.0f} | "
              f"{'' if lds <= 0 else format(v['SQ_LDS_BANK_CONFLICT'] / lds, '.3f')} |")
    return 0


ISSUE_COUNTERS = ["SQ_VALU_MFMA_BUSY_CYCLES", "SQ_VALU_MFMA_COEXEC_CYCLES", "SQ_VMEM_TA_CMD_FIFO_FULL",
                  "SQ_VMEM_TA_ADDR_FIFO_FULL", "SQ_INSTS_VALU", "SQ_INSTS_MFMA", "SQ_INSTS_LDS", "GRBM_GUI_ACTIVE"]


def cmd_issue(ns) -> int:
    """What the SIMDs issue and what holds the memory instructions back: matrix pipe busy, matrix and vector pipe
    busy at once, cycles with the address unit's queues full, instruction counts per launch."""
    scope = ["--no-extra"] if ns.all_ops else ["--form", ns.form, "--step-only"]
    bench_args = ["--workload", ns.workload] + scope + ["--no-cpu", "--steps", str(ns.steps), "--warmup", str(ns.warmup)]
    decode = ns.workload == "c5"
    d, line, shown = run_profiler(f"issue_{ns.workload}", ["--pmc"] + ISSUE_COUNTERS, bench_args, ns.timeout)
    path = find_csv(d, "counter_collection.csv")
    per = {c: counter_rows(path, c) for c in ISSUE_COUNTERS}
    keys = collections.defaultdict(lambda: collections.defaultdict(float))
    names = collections.defaultdict(set)
    for c, rows in per.items():
        for name, vals in rows.items():
            key = key_of(name, decode)
            if key is None or key == "copy":
                continue
            keys[key][c] += sum(vals)
            keys[key]["n_" + c] = max(keys[key]["n_" + c], len(vals))
            names[key].add(name[:70])
    print(f"# Issue counters of the kernels of `bench.py --workload {ns.workload} {' '.join(scope)}`\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout):\n")
    print(f"```\npython3 bench_profiles.py issue --workload {ns.workload}"
          f"{' --all-ops' if ns.all_ops else ' --form ' + ns.form}\n  -> {shown}\n```\n")
    print_sources(line)
    print("Shares are of all SIMD cycles of an op's launches (`GRBM_GUI_ACTIVE` / 8 XCDs x 1024 SIMDs); the queue "
          "counters are per SIMD as well.  Instruction counts are per launch, summed over all waves.\n")
    print("| op (key in the bench line) | kernels | matrix pipe busy | matrix and vector pipe busy at once | "
          "address unit's command queue full | address unit's address queue full | VALU instructions (incl. MFMA), M | "
          "MFMA instructions, M | LDS instructions, M |\n|---|---|---|---|---|---|---|---|---|")
    for key, v in keys.items():
        simd = v["GRBM_GUI_ACTIVE"] / 8 * 1024
        if simd <= 0:
            continue
        n = max(v["n_SQ_INSTS_VALU"], 1)
        print(f"| `{key}` | {'; '.join(sorted(names[key]))} | {v['SQ_VALU_MFMA_BUSY_CYCLES'] / simd:.3f} | "
              f"{v['SQ_VALU_MFMA_COEXEC_CYCLES'] / simd:.3f} | {v['SQ_VMEM_TA_CMD_FIFO_FULL'] / simd:.3f} | "
              f"{v['SQ_VMEM_TA_ADDR_FIFO_FULL'] / simd:.3f} | {v['SQ_INSTS_VALU'] / n / 1e6:.2f} | "
              f"{v['SQ_INSTS_MFMA'] / n / 1e6:.2f} | {v['SQ_INSTS_LDS'] / n / 1e6:.2f} |")
    return 0


# three runs of at most four L2 (TCC) counters each, plus the cycle count that turns stalls into shares
MEMSYS_RUNS = [
    ["TCC_REQ_sum", "TCC_HIT_sum", "TCC_MISS_sum", "GRBM_GUI_ACTIVE"],
    ["TCC_EA0_RDREQ_sum", "TCC_EA0_WRREQ_sum", "TCC_EA0_WRREQ_64B_sum", "TCC_EA0_RDREQ_32B_sum", "GRBM_GUI_ACTIVE"],
    ["TCC_EA0_WRREQ_STALL_sum", "TCC_TOO_MANY_EA_WRREQS_STALL_sum", "TCC_TAG_STALL_sum",
     "TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum", "GRBM_GUI_ACTIVE"],
]


def cmd_memsys(ns) -> int:
    """What the L2 and its memory interface see: hit rate, requests that go on to memory by size, and the cycles a
    channel could not send (summed over the 16 channels of each of the 8 XCDs, so a share of 1.0 would be every
    channel blocked all the time)."""
    scope = ["--no-extra"] if ns.all_ops else ["--form", ns.form, "--step-only"]
    bench_args = ["--workload", ns.workload] + scope + ["--no-cpu", "--steps", str(ns.steps), "--warmup", str(ns.warmup)]
    decode = ns.workload == "c5"
    keys = collections.defaultdict(lambda: collections.defaultdict(float))
    shown_all = []
    for i, counters in enumerate(MEMSYS_RUNS):
        d, line, shown = run_profiler(f"memsys{i}_{ns.workload}", ["--pmc"] + counters, bench_args, ns.timeout)
        shown_all.append(shown)
        path = find_csv(d, "counter_collection.csv")
        for c in counters:
            for name, vals in counter_rows(path, c).items():
                key = key_of(name, decode)
                if key is None or key == "copy":
                    continue
                tag = c if c != "GRBM_GUI_ACTIVE" else f"cycles{i}"
                keys[key][tag] += sum(vals)
                keys[key]["n_" + tag] = max(keys[key]["n_" + tag], len(vals))
    print(f"# L2 and memory-interface counters of the kernels of `bench.py --workload {ns.workload} {' '.join(scope)}`\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout):\n")
    print(f"```\npython3 bench_profiles.py memsys --workload {ns.workload}"
          f"{' --all-ops' if ns.all_ops else ' --form ' + ns.form}")
    for sh in shown_all:
        print(f"  -> {sh}")
    print("```\n")
    print_sources(line)
    print("Requests are per launch, in millions.  Requests to memory: reads of 32 / 64 bytes (the rest are 128-byte "
          "reads), writes of 64 bytes (the rest 32).  Stall shares: cycles summed over the L2 channels divided by "
          "128 channels x the launch's cycles (`GRBM_GUI_ACTIVE` counts the cycles of all 8 XCDs).\n")
    print("| op (key in the bench line) | L2 requests, M | L2 hit rate | reads to memory, M (32-byte ones) | "
          "writes to memory, M (64-byte ones) | write requests held back | too many writes outstanding | tag stall | "
          "read credits to DRAM exhausted |\n|---|---|---|---|---|---|---|---|---|")
    for key, v in keys.items():
        n0, n1 = max(v["n_TCC_REQ_sum"], 1), max(v["n_TCC_EA0_RDREQ_sum"], 1)
        chan_cycles = v["cycles2"] / 8 * 128
        if chan_cycles <= 0:
            continue
        hit = v["TCC_HIT_sum"] / max(v["TCC_HIT_sum"] + v["TCC_MISS_sum"], 1.0)
        print(f"| `{key}` | {v['TCC_REQ_sum'] / n0 / 1e6:.2f} | {hit:.3f} | {v['TCC_EA0_RDREQ_sum'] / n1 / 1e6:.2f} "
              f"({v['TCC_EA0_RDREQ_32B_sum'] / n1 / 1e6:.2f}) | {v['TCC_EA0_WRREQ_sum'] / n1 / 1e6:.2f} "
              f"({v['TCC_EA0_WRREQ_64B_sum'] / n1 / 1e6:.2f}) | {v['TCC_EA0_WRREQ_STALL_sum'] / chan_cycles:.3f} | "
              f"{v['TCC_TOO_MANY_EA_WRREQS_STALL_sum'] / chan_cycles:.3f} | {v['TCC_TAG_STALL_sum'] / chan_cycles:.3f} | "
              f"{v['TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum'] / chan_cycles:.3f} |")
    return 0


def cmd_yardstick(ns) -> int:
    """bench.py --copy-yardstick (no profiler: event timings) as a table: what a kernel that only moves the bytes
    reaches in each access pattern of the library's memory-bound kernels."""
    cmd = ["python3", os.path.join(ROOT, "bench.py"), "--copy-yardstick", "--steps", str(ns.steps)]
    proc = subprocess.run(cmd, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=ns.timeout)
    if proc.returncode != 0:
        sys.stderr.write(proc.stderr[-3000:])
        raise SystemExit(f"bench.py exited with {proc.returncode}")
    line = [json.loads(ln) for ln in proc.stdout.splitlines() if ln.startswith("{")][-1]
    y = line["yardsticks"]
    print("# Bandwidth yardsticks: kernels that only move bytes, in the access patterns of the memory-bound kernels\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout; HIP-event timings, no profiler):\n")
    print(f"```\npython3 bench_profiles.py yardstick\n  -> python3 bench.py --copy-yardstick --steps {ns.steps}\n```\n")
    print_sources(line)
    print("All figures are GB/s of the bytes the pattern moves (a copy and an in-place or out-of-place pass move every "
          "byte twice: once in, once out); `_nt` = non-temporal loads and stores.  Kernels: "
          "`energonai_amd/csrc/yardstick.hip` (`en_stream_yardstick`, `en_prefix_yardstick`) and `copy_kernel` "
          "(`en_copy_bytes`).\n")
    print("## One contiguous range (depad, the transposes, LayerNorm, the decode kernels' cache reads)\n")
    cols = ["copy", "copy_nt", "inplace", "inplace_nt", "read", "read_nt", "write", "write_nt"]
    print("| size | " + " | ".join(cols) + " | `en_copy_bytes` |\n|---|" + "---|" * (len(cols) + 1))
    plain = {k: v["GBps"] for k, v in line["sizes"].items()}
    for size, row in y["stream"].items():
        print(f"| {size} | " + " | ".join(f"{row[c]:.0f}" for c in cols) + f" | {plain.get(size, float('nan')):.0f} |")
    print("\n`en_copy_bytes` (the counter-calibration copy) at its own sizes: " +
          ", ".join(f"{k} {v:.0f}" for k, v in plain.items()) + " GB/s.\n")
    print("## Causal prefixes of a score tensor (row q of a unit: q + 1 fp16 scores; rows below the sequence length only)\n")
    print("`inplace`: read and written back (scale_mask_softmax without a tail); `write`: written only (QK^T); `read`: read "
          "only (PV); `out_of_place`: read from one tensor, written to another.  `padded` = `[B,H,S,S]`, `packed` = the "
          "packed causal layout.  c3: 16 sequences of 142..1014 tokens, 56 heads; c4: 16 of 360..2019, 12 heads.\n")
    cols = [f"{m}{t}" for m in ("inplace", "write", "read", "out_of_place") for t in ("", "_nt")]
    print("| lengths, layout | " + " | ".join(cols) + " |\n|---|" + "---|" * len(cols))
    for name, row in y["prefix"].items():
        print(f"| {name.replace('_', ', ')} | " + " | ".join(f"{row[c]:.0f}" for c in cols) + " |")
    print("\n## The same prefixes read the way PV walks them (`prefix_tile_walk_kernel`)\n")
    print("One workgroup per tile of 128 rows, moving along the keys in steps of 128 bytes per row (64 fp16 keys, the key "
          "tile of the attention kernels) or 256 bytes, every row as far as its prefix goes, the next step's loads in "
          "flight while this step's are consumed; no LDS traffic, no arithmetic.  `3 per CU`: 48 KB of idle LDS per "
          "workgroup, the occupancy of the attention kernels.  The bytes are those of the `read` column above.\n")
    cols = [f"{m}{t}" for m in ("read_tile_walk", "read_tile_walk_3_per_cu", "read_tile_walk_256B",
                                "read_tile_walk_256B_3_per_cu") for t in ("", "_nt")]
    head = [("256 B" if "256B" in c else "128 B") + (", 3 per CU" if "3_per_cu" in c else "") +
            (", non-temporal" if c.endswith("_nt") else "") for c in cols]
    print("| lengths, layout | " + " | ".join(head) + " |\n|---|" + "---|" * len(cols))
    for name, row in y["prefix"].items():
        print(f"| {name.replace('_', ', ')} | " + " | ".join(f"{row[c]:.0f}" for c in cols) + " |")
    return 0


def cmd_decode(ns) -> int:
    """bench.py --decode-sizes (no profiler: event timings) as a table."""
    cmd = ["python3", os.path.join(ROOT, "bench.py"), "--decode-sizes", "--steps", str(ns.steps)]
    proc = subprocess.run(cmd, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=ns.timeout)
    if proc.returncode != 0:
        sys.stderr.write(proc.stderr[-3000:])
        raise SystemExit(f"bench.py exited with {proc.returncode}")
    line = [json.loads(ln) for ln in proc.stdout.splitlines() if ln.startswith("{")][-1]
    print("# Single-pass decode attention from one sequence to 64: one workgroup per unit, shared keys, pages\n")
    print("Command (MI355X box, repo root; the summary below is this command's stdout; HIP-event timings, no profiler):\n")
    print(f"```\npython3 bench_profiles.py decode\n  -> python3 bench.py --decode-sizes --steps {ns.steps}\n```\n")
    print_sources(line)
    print(f"{line['heads']} heads of {line['size_per_head']} channels, {line['dtype']}, every cache full; a (batch, head) "
          "unit is one workgroup of 1024 lanes unless its keys are shared.  `as called`: what `en_decode_attn` does when "
          "the caller brings the workspace (fewer than 512 units and at least 1024 cached positions: the keys of a unit "
          "go to several workgroups and a second small kernel combines them; its time is included).  `pages`: "
          f"`en_decode_attn_paged` on the same contents in pages of {line['page']} positions with shuffled ids.  "
          "TB/s = K and V bytes of the cached positions over the time.\n")
    print("| sequences | cached positions | units | K + V, MB | workgroups per unit | one workgroup per unit, us (TB/s) | "
          "as called, us (TB/s) | pages, us (TB/s) |\n|---|---|---|---|---|---|---|---|")
    cell = lambda r: f"{r['us']:.1f} ({r['GBps'] / 1e3:.2f})"
    for r in line["rows"]:
        print(f"| {r['batch']} | {r['cached_positions']} | {r['units']} | {r['cache_MB']:.0f} | {r['shares_per_unit']} | "
              f"{cell(r['one_workgroup_per_unit'])} | {cell(r['as_called'])} | {cell(r['paged'])} |")
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    p = sub.add_parser("decode")
    p.add_argument("--steps", type=int, default=20)
    p.add_argument("--timeout", type=int, default=300)
    p.add_argument("--raw-dir", default=None)
    p.set_defaults(fn=cmd_decode)
    p = sub.add_parser("yardstick")
    p.add_argument("--steps", type=int, default=10)
    p.add_argument("--timeout", type=int, default=300)
    p.add_argument("--raw-dir", default=None)
    p.set_defaults(fn=cmd_yardstick)
    for name, fn in (("trace", cmd_trace), ("traffic", cmd_traffic), ("counters", cmd_counters), ("issue", cmd_issue),
                     ("memsys", cmd_memsys)):
        p = sub.add_parser(name)
        p.add_argument("--workload", default="c3", choices=["c1", "c2", "c3", "c4", "c5"])
        p.add_argument("--form", default="default", choices=["default", "three_kernel"],
                       help="which form of the step bench.py times (its --form)")
        p.add_argument("--steps", type=int, default=20)
        p.add_argument("--warmup", type=int, default=5)
        p.add_argument("--timeout", type=int, default=300, help="seconds allowed for each rocprofv3 run")
        p.add_argument("--raw-dir", default=None, help="directory for rocprofv3's raw output (default: a temporary one)")
        if name in ("counters", "issue", "memsys"):
            p.add_argument("--all-ops", action="store_true", help="every op of the bench line, not the step alone")
        p.set_defaults(fn=fn)
    ns = ap.parse_args(argv)
    global OUT
    OUT = ns.raw_dir
    return ns.fn(ns)


if __name__ == "__main__":
    sys.exit(main())
