"""rocprofv3 passes over one bench.py workload and their summary.

    python -m deca_amd.arch.profile run WORKLOAD [--out DIR]        # on the GPU box
    python -m deca_amd.arch.profile summarise WORKLOAD [--out DIR]  # anywhere

`run` starts the profiler passes as child processes, one pass per run (the
counters of a pass must fit the hardware, and counter passes are never mixed
with traces):

    trace   --kernel-trace --stats                       100 steps
    fetch   --pmc FETCH_SIZE                             20 steps
    write   --pmc WRITE_SIZE                             20 steps
    sq      --pmc SQ_* GRBM_GUI_ACTIVE (matrix kernels)  20 steps
    board   no profiler: bench.py --power 4 (shader clock and socket power, sampled once a
            second while the kernel repeats)

each over `python3 bench.py --workload WORKLOAD --no-extra --no-cpu`.
`summarise` turns their CSV files into `profiles/<kernel>_<workload>.md` and
records the traffic figure bench.py reports in `deca_amd/measured_traffic.json`.

The role of the reference's pasted-in nsight / microbenchmark figures
(arch/H20.py:35-60): the numbers the hardware model and the cost model are
judged against, here with the commands that make them.
"""

from __future__ import annotations

import argparse
import collections
import csv
import json
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROOT = os.path.dirname(PKG)

KERNEL_OF = {"rmsnorm": "rowwise", "softmax": "rowwise", "gemm": "gemm", "fa": "flash_attn"}
SQ_COUNTERS = ("SQ_VALU_MFMA_BUSY_CYCLES", "SQ_INSTS_MFMA", "SQ_INSTS_VALU", "SQ_ACTIVE_INST_VALU",
               "SQ_VALU_MFMA_COEXEC_CYCLES", "SQ_INSTS_LDS", "SQ_LDS_BANK_CONFLICT", "GRBM_GUI_ACTIVE")
NOMINAL_GHZ = 2.4
SIMDS = 256 * 4
XCDS = 8
# FETCH_SIZE reports half of the bytes read, WRITE_SIZE the bytes written (KiB per
# dispatch): measured against a copy kernel of 128 MiB in / 128 MiB out
# (`python -m deca_amd.arch.ceilings --copy-only` under the same two counter passes).
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0
# Below this dispatch length the GRBM_GUI_ACTIVE window (which opens before the first
# wave and closes after the last) is no measure of the kernel's own cycles, and no clock
# or busy share is derived from it.
MIN_NS_FOR_CLOCK = 100_000


def kernel_of(workload: str) -> str:
    return KERNEL_OF[workload.split("_")[0]]


def passes(workload: str, kernel_config: str | None = None) -> dict:
    """name -> (rocprofv3 options, bench.py options) of the profiler passes; with
    `kernel_config`, over that configuration instead of the stored winner."""
    bench = ["--workload", workload, "--no-extra", "--no-cpu", "--full-out", ""]
    if kernel_config:
        bench += ["--kernel-config", kernel_config]
    short = bench + ["--steps", "20", "--warmup", "2"]
    out = {
        "trace": (["--kernel-trace", "--stats"], bench + ["--steps", "100", "--warmup", "10"]),
        "fetch": (["--pmc", "FETCH_SIZE"], short),
        "write": (["--pmc", "WRITE_SIZE"], short),
    }
    if kernel_of(workload) != "rowwise":
        out["sq"] = (["--pmc", *SQ_COUNTERS], short)
    out["board"] = (None, short + ["--power", "4"])
    return out


def command(workload: str, name: str, out_dir: str, kernel_config: str | None = None) -> list:
    prof, bench = passes(workload, kernel_config)[name]
    if prof is None:
        return ["python3", os.path.join(ROOT, "bench.py"), *bench]
    return ["rocprofv3", *prof, "-d", os.path.join(out_dir, name), "-o", "out", "--output-format", "csv",
            "--", "python3", os.path.join(ROOT, "bench.py"), *bench]


def run(workload: str, out_dir: str, timeout_s: int = 200, kernel_config: str | None = None) -> None:
    """Runs the passes one after the other; stops at the first that fails."""
    os.makedirs(out_dir, exist_ok=True)
    env = dict(os.environ, TMPDIR="/tmp")
    for name in passes(workload, kernel_config):
        cmd = command(workload, name, out_dir, kernel_config)
        print("[profile]", " ".join(cmd), flush=True)
        with open(os.path.join(out_dir, f"{name}.log"), "w") as log:
            done = subprocess.run(cmd, cwd="/tmp", env=env, stdout=log, stderr=subprocess.STDOUT,
                                  timeout=timeout_s)
        if done.returncode != 0:
            raise SystemExit(f"pass {name} of {workload} failed with status {done.returncode}")


# ---------------------------------------------------------------------------
# reading the profiler's CSV files
# ---------------------------------------------------------------------------
def _mean(values):
    values = list(values)
    return sum(values) / len(values)


def _rows(path: str) -> list:
    with open(path, newline="") as f:
        return list(csv.DictReader(f))


def bench_record(log_path: str):
    """The JSON line bench.py printed in a pass (None when there is none)."""
    rec = None
    with open(log_path) as f:
        for line in f:
            if line.startswith("{"):
                rec = json.loads(line)
    return rec


def event_timed_durations(trace_rows: list, first: int, count: int) -> list:
    """Durations (ns) of the launches bench.py timed: `count` launches of the kernel under
    test from its `first` one on (the record's `roofline.timed_launches`; spin-up and warm-up
    launches come before them, the row-wise pass over a single buffer set and the GEMM's
    pass on N(0,1) operands after)."""
    mine = sorted((r for r in trace_rows if r["Kernel_Name"].startswith("deca_main")),
                  key=lambda r: int(r["Start_Timestamp"]))
    durs = [int(r["End_Timestamp"]) - int(r["Start_Timestamp"]) for r in mine]
    if not 0 <= first <= first + count <= len(durs):
        raise ValueError(f"the trace holds {len(durs)} launches, the record times {first}..{first + count}")
    return durs[first:first + count]


def counter_means(counter_rows: list, kernel_prefix: str | None = None) -> dict:
    """kernel name -> counter name -> (mean value, dispatches), optionally only kernels
    whose name starts with `kernel_prefix`."""
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    for r in counter_rows:
        if kernel_prefix is None or r["Kernel_Name"].startswith(kernel_prefix):
            agg[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return {k: {c: (_mean(v), len(v)) for c, v in cs.items()} for k, cs in agg.items()}


def traffic_bytes(fetch_kib: float, write_kib: float) -> int:
    """L2 <-> fabric bytes per dispatch from the two counters (Infinity Cache hits
    included: an upper bound of the HBM traffic)."""
    return int(round((fetch_kib * FETCH_SCALE + write_kib * WRITE_SCALE) * 1024))


def matrix_pipe(sq_rows: list) -> dict:
    """Derived figures of the `sq` pass for `deca_main`.

    `peak_share` = MFMA busy cycles / (SIMDs x duration x nominal clock) needs no cycle
    count of the dispatch.  `clock_ghz` and `busy` (busy cycles / shader cycles) rest on
    GRBM_GUI_ACTIVE / 8 XCDs as the dispatch's cycle count and are None for dispatches
    shorter than MIN_NS_FOR_CLOCK, where that window is dominated by what surrounds the
    kernel (a 19 us dispatch read 2.97 GHz on a 2.4 GHz part that way)."""
    rows = [r for r in sq_rows if r["Kernel_Name"].startswith("deca_main")]
    per = collections.defaultdict(list)
    dur = {}
    for r in rows:
        per[r["Counter_Name"]].append(float(r["Counter_Value"]))
        dur[r["Dispatch_Id"]] = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
    m = {k: _mean(v) for k, v in per.items()}
    ns = _mean(dur.values())
    busy_cycles = m["SQ_VALU_MFMA_BUSY_CYCLES"]
    out = {
        "duration_ns": ns,
        "mfma": m["SQ_INSTS_MFMA"],
        "peak_share": busy_cycles / (SIMDS * ns * NOMINAL_GHZ),
        "coexec": m["SQ_VALU_MFMA_COEXEC_CYCLES"] / busy_cycles,
        "valu_per_mfma": m["SQ_INSTS_VALU"] / m["SQ_INSTS_MFMA"],
        "lds_per_mfma": m["SQ_INSTS_LDS"] / m["SQ_INSTS_MFMA"],
        "bank_conflict_cycles": m["SQ_LDS_BANK_CONFLICT"],
        "clock_ghz": None, "busy": None, "cycles": None,
    }
    if ns >= MIN_NS_FOR_CLOCK:
        cycles = m["GRBM_GUI_ACTIVE"] / XCDS
        out.update(cycles=cycles, clock_ghz=cycles / ns, busy=busy_cycles / (SIMDS * cycles))
    return out


# ---------------------------------------------------------------------------
# the summary
# ---------------------------------------------------------------------------
def summary_text(workload: str, out_dir: str, kernel_config: str | None = None) -> tuple:
    """(markdown text, entry for measured_traffic.json) from the passes' output."""
    kern = kernel_of(workload)
    rowwise = kern == "rowwise"
    rec = bench_record(os.path.join(out_dir, "trace.log"))
    stats = _rows(os.path.join(out_dir, "trace", "out_kernel_stats.csv"))
    trace = _rows(os.path.join(out_dir, "trace", "out_kernel_trace.csv"))
    steps = int(rec["steps"])
    ev = event_timed_durations(trace, *rec["roofline"]["timed_launches"])
    fetch = counter_means(_rows(os.path.join(out_dir, "fetch", "out_counter_collection.csv")))
    write = counter_means(_rows(os.path.join(out_dir, "write", "out_counter_collection.csv")))

    def rel(cmd):
        words = [f"'{w}'" if ("," in w or not w) else w for w in cmd]
        return " ".join(words).replace(out_dir, "<out>").replace(ROOT + os.sep, "")

    extra = f" --kernel-config '{kernel_config}'" if kernel_config else ""
    t = [f"# rocprofv3 summary: `{kern}.hip` on workload `{workload}`"
         + (f", configuration `{kernel_config}`" if kernel_config else ""), "",
         f"Made by `python -m deca_amd.arch.profile run {workload}{extra}` and `... summarise "
         f"{workload}{extra}` on a 1-GPU MI355X box; the passes it runs (from `/tmp`, `TMPDIR=/tmp`):",
         "", "```"]
    t += [rel(command(workload, name, out_dir, kernel_config)) for name in passes(workload, kernel_config)]
    t += ["```", "", "## Kernel trace statistics (top kernels)", "",
          "| kernel | calls | avg ns | min ns | max ns | % of GPU time |", "|---|---|---|---|---|---|"]
    for r in stats[:4]:
        t.append(f"| `{r['Name'][:70]}` | {r['Calls']} | {float(r['AverageNs']):.0f} | {r['MinNs']} | "
                 f"{r['MaxNs']} | {float(r['Percentage']):.2f} |")
    t += ["", "`deca_main` is the kernel under test; the others are torch's input generators. The "
          "statistics cover every launch of the run: 0.3 s of untimed spin-up (clocks still ramping), "
          f"the warm-up steps, the {steps} timed steps (host clock and events around the same launches"
          + (", rotating buffers)" if rowwise else ")")
          + (f", then {steps} more over one buffer set" if rowwise else "")
          + (", then the passes on N(0,1) operands" if kern == "gemm" else "") + ".", "",
          f"From `out_kernel_trace.csv` of the same run, the {len(ev)} timed launches alone: average "
          f"{_mean(ev):.0f} ns (min {min(ev)}, max {max(ev)}); bench.py reports kernel_us = "
          f"{rec['roofline']['kernel_us']:.2f} for them (event span / {len(ev)}: it includes the gaps "
          "between consecutive launches).", "",
          "## bench.py line of the same run (HIP-event timing on the launch stream)", "", "```",
          json.dumps(rec), "```", "", "## L2 <-> fabric traffic per dispatch (KiB as reported)", "",
          "| kernel | FETCH_SIZE mean | WRITE_SIZE mean | dispatches |", "|---|---|---|---|"]
    for k, cs in fetch.items():
        fv, n = cs["FETCH_SIZE"]
        wv = write.get(k, {}).get("WRITE_SIZE", (0.0, 0))[0]
        t.append(f"| `{k[:70]}` | {fv:.1f} | {wv:.1f} | {n} |")
    mine_f = next(cs["FETCH_SIZE"][0] for k, cs in fetch.items() if k.startswith("deca_main"))
    mine_w = next(cs["WRITE_SIZE"][0] for k, cs in write.items() if k.startswith("deca_main"))
    total = traffic_bytes(mine_f, mine_w)
    work = rec["roofline"]["all"][workload]["work"]
    t += ["", f"`deca_main`: {FETCH_SCALE:.1f} x FETCH_SIZE + {WRITE_SCALE:.1f} x WRITE_SIZE = "
          f"{total / 1e6:.1f} MB per launch"
          + (f" against {work / 1e6:.1f} MB of algorithmic bytes ({total / work:.3f}x)." if rowwise else "."),
          "Scale factors: against a copy kernel of 128 MiB in / 128 MiB out FETCH_SIZE reports half of "
          "the bytes read and WRITE_SIZE the bytes written "
          "(`profiles/traffic_counter_calibration_copy_128mib.md`). Both count L2 <-> data-fabric "
          "traffic (Infinity Cache hits included), an upper bound of HBM traffic."]
    sq_path = os.path.join(out_dir, "sq", "out_counter_collection.csv")
    if os.path.exists(sq_path):
        mp = matrix_pipe(_rows(sq_path))
        m16 = "mfma=16" in rec["config"]["kernel_config"]
        form = "16x16x32, 16 clocks each" if m16 else "32x32x16, 32 clocks each"
        t += ["", "## Matrix pipe of `deca_main` (the `sq` pass)", "", "| quantity | value |", "|---|---|",
              f"| dispatch duration under the counters | {mp['duration_ns'] / 1e3:.1f} us |",
              f"| SQ_INSTS_MFMA ({form}) | {mp['mfma']:.4g} |",
              "| SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs x duration x 2.4 GHz) = share of the "
              f"2.5 PFLOP/s peak | {100 * mp['peak_share']:.1f} % |"]
        if mp["clock_ghz"] is not None:
            t += [f"| GRBM_GUI_ACTIVE / 8 XCDs = shader cycles per dispatch | {mp['cycles']:.4g} |",
                  f"| average shader clock during the dispatch | {mp['clock_ghz']:.2f} GHz "
                  f"({NOMINAL_GHZ} GHz nominal) |",
                  f"| MFMA busy cycles / (1024 SIMDs x shader cycles) = matrix pipe busy | "
                  f"{100 * mp['busy']:.1f} % |"]
        else:
            t.append(f"| shader clock, busy share of the cycles | not derived: the dispatch is shorter than "
                     f"{MIN_NS_FOR_CLOCK // 1000} us and GRBM_GUI_ACTIVE also counts what surrounds it |")
        t += [f"| SQ_VALU_MFMA_COEXEC_CYCLES / MFMA busy cycles (vector ALU running beside the matrix "
              f"pipe) | {100 * mp['coexec']:.1f} % |",
              f"| SQ_INSTS_VALU (includes MFMA) per MFMA | {mp['valu_per_mfma']:.2f} |",
              f"| SQ_INSTS_LDS per MFMA | {mp['lds_per_mfma']:.2f} |",
              f"| SQ_LDS_BANK_CONFLICT cycles | {mp['bank_conflict_cycles']:.4g} |"]
    board_log = os.path.join(out_dir, "board.log")
    board = bench_record(board_log) if os.path.exists(board_log) else None
    if board and "socket_w" in board["roofline"]:
        rf = board["roofline"]
        clk = rf.get("sclk_mhz", [0, 0])
        t += ["", "## Board state while the kernel repeats (the `board` pass: rocm-smi / amd-smi, one "
              "sample a second for 4 s)", "",
              f"Shader clock {clk[0]:.0f}-{clk[1]:.0f} MHz, socket power {rf['socket_w'][0]:.0f}-"
              f"{rf['socket_w'][1]:.0f} W; the launches timed just before ran at {rf['achieved']:.0f} "
              f"{rf['unit']}."]
    entry = {"config": rec["config"]["kernel_config"], "fetch_size_kib": round(mine_f, 1),
             "write_size_kib": round(mine_w, 1), "fetch_scale": FETCH_SCALE, "write_scale": WRITE_SCALE,
             "traffic_bytes": total}
    return "\n".join(t) + "\n", entry


def summarise(workload: str, out_dir: str, profiles_dir: str | None = None,
              traffic_path: str | None = None, kernel_config: str | None = None,
              tag: str | None = None) -> str:
    """Writes the summary; the traffic table only takes figures of the stored winners (a
    run over another `kernel_config` is written as `..._<tag>.md` and recorded nowhere)."""
    text, entry = summary_text(workload, out_dir, kernel_config)
    profiles_dir = profiles_dir or os.path.join(ROOT, "profiles")
    name = f"{kernel_of(workload)}_{workload}" + (f"_{tag}" if kernel_config else "")
    path = os.path.join(profiles_dir, name + ".md")
    with open(path, "w") as f:
        f.write(text)
    if kernel_config:
        return path
    traffic_path = traffic_path or os.path.join(PKG, "measured_traffic.json")
    table = {"workloads": {}}
    if os.path.exists(traffic_path):
        with open(traffic_path) as f:
            table = json.load(f)
    table.setdefault("workloads", {})[workload] = entry
    with open(traffic_path, "w") as f:
        json.dump(table, f, indent=1)
        f.write("\n")
    return path


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("action", choices=["run", "summarise"])
    ap.add_argument("workload")
    ap.add_argument("--out", default=None, help="directory of the passes' output "
                                                "(default profile_out/prof_<workload>[_<tag>])")
    ap.add_argument("--kernel-config", default=None, metavar="TEXT",
                    help="profile this configuration instead of the stored winner")
    ap.add_argument("--tag", default="variant", help="with --kernel-config: suffix of the summary's name")
    args = ap.parse_args(argv)
    default = f"prof_{args.workload}" + (f"_{args.tag}" if args.kernel_config else "")
    out_dir = os.path.abspath(args.out or os.path.join(ROOT, "profile_out", default))
    if args.action == "run":
        run(args.workload, out_dir, kernel_config=args.kernel_config)
    else:
        print("wrote", summarise(args.workload, out_dir, kernel_config=args.kernel_config, tag=args.tag))


if __name__ == "__main__":
    sys.exit(main())
