#!/usr/bin/env python3
"""Benchmark of the tuned kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra]

A step is one launch of the workload's kernel over one batch of synthetic
input already resident in HBM.  Prints ONE JSON line, last on standard output:
the headline workload's throughput (`value`), its roofline fraction measured
with HIP events on the launch stream, the torch-CPU baseline timed on this
box's host cores, and -- unless --no-extra -- the same figures for the other
benchmark configurations in compact form under roofline.all and
cpu_baseline.all.  The full per-workload records go to --full-out.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0
MALL_BYTES = 256 * 1024 * 1024


def _cfg(operator, shape, dtype="float16", causal=False):
    """The stored winner of a tuning run for this workload (GEMM: of the run on the
    benchmark's U(-1,1) operands)."""
    from deca_amd import tuned

    key = tuned.make_key(operator, shape, dtype, "gfx950", causal,
                         "uniform" if operator == "GEMM" else "normal")
    cfg = tuned.lookup(key)
    if cfg is None:
        raise KeyError(f"no tuned config for {key}: run the matching test_*.py driver with --cache")
    return cfg


# name -> description of the workload (the benchmark configurations)
def workloads():
    w = {}
    for name, (op, M, N, dtype) in {
        "rmsnorm_bf16_16384x4096": ("rmsnorm", 16384, 4096, "bfloat16"),
        "softmax_fp16_16384x4096": ("softmax", 16384, 4096, "float16"),
        "rmsnorm_fp16_8192x8192": ("rmsnorm", 8192, 8192, "float16"),
    }.items():
        w[name] = {"kind": "rowwise", "op": op, "M": M, "N": N, "dtype": dtype,
                   "cfg": _cfg(op, (M, N), dtype)}
    for n in (2048, 4096, 8192, 12288, 16384):
        w[f"gemm_fp16_{n}"] = {"kind": "gemm", "M": n, "N": n, "K": n, "dtype": "float16",
                               "cfg": _cfg("GEMM", (n, n, n))}
    w["gemm_bf16_8192"] = {"kind": "gemm", "M": 8192, "N": 8192, "K": 8192, "dtype": "bfloat16",
                           "cfg": _cfg("GEMM", (8192, 8192, 8192), "bfloat16")}
    for D in (128, 64):
        for causal in (False, True):
            name = f"fa_fp16_b4h16s4096d{D}" + ("_causal" if causal else "")
            w[name] = {"kind": "fa", "B": 4, "H": 16, "S": 4096, "D": D, "causal": causal,
                       "cfg": _cfg("flash_attn", (4, 16, 4096, 4096, D), "float16", causal)}
    for k, v in w.items():
        v["name"] = k
    return w


DEFAULT_WORKLOAD = "rmsnorm_bf16_16384x4096"
SPIN_UP_SECONDS = 0.3
POWER_SECONDS = 0  # --power: seconds of board-state sampling per workload


def _board(kern, sets):
    """Shader clock and socket power (rocm-smi / amd-smi, one sample a second) while the
    kernel repeats over `sets`; {} unless --power was given."""
    if POWER_SECONDS <= 0:
        return {}
    import io
    import re

    from deca_amd.arch import ceilings

    buf = io.StringIO()
    ceilings.sample_while(lambda: [kern(*sets[i % len(sets)]) for i in range(50)], "board", buf,
                           seconds=POWER_SECONDS + 1)
    lines = buf.getvalue().splitlines()[1:]  # the first second still ramps
    for line in lines:
        print(f"[bench]   {line}", file=sys.stderr, flush=True)
    mhz = [float(v) for line in lines for v in re.findall(r"\((\d+)Mhz\)", line)[:1]]
    watts = [float(v) for line in lines for v in re.findall(r"SOCKET_POWER:\s*(\d+)", line)]
    out = {}
    if mhz:
        out["sclk_mhz"] = [min(mhz), max(mhz)]
    if watts:
        out["socket_w"] = [min(watts), max(watts)]
    return out


def _spec(wl):
    if wl["kind"] == "rowwise":
        from deca_amd.kernels.rowwise_hip import make_rowwise

        return make_rowwise(wl["op"], wl["M"], wl["N"], wl["dtype"], wl["cfg"], 1e-6)
    if wl["kind"] == "gemm":
        from deca_amd.kernels.gemm_hip import make_gemm_tc

        return make_gemm_tc(wl["M"], wl["N"], wl["K"], wl["cfg"], wl["dtype"])
    if wl["kind"] == "fa":
        from deca_amd.kernels.flash_attn_hip import make_flash_attn_fwd

        return make_flash_attn_fwd(wl["B"], wl["H"], wl["S"], wl["S"], wl["D"], wl["cfg"], None,
                                   wl["causal"])
    raise ValueError(wl["kind"])


def bench_specs():
    """Kernel specialisations this script loads (compiled ahead by the build step)."""
    return [_spec(wl) for wl in workloads().values()]


# ---------------------------------------------------------------------------
# CPU baseline: torch's CPU operator on a bounded sample of the same workload
# ---------------------------------------------------------------------------
def cpu_baseline(wl):
    import torch

    from oracle import baseline as ob

    t0 = time.perf_counter()
    res = ob.time_cpu(wl, torch.get_num_threads())
    print(f"[bench]   cpu baseline of {wl['name']}: {res['value']:.3g} {res['unit']} on "
          f"{res['cores']} threads in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    return res


# ---------------------------------------------------------------------------
# one workload
# ---------------------------------------------------------------------------
def run_rowwise(wl, steps, warmup, with_cpu):
    import torch

    from deca_amd.kernels.rowwise_bench import make_inputs, rowwise_bytes
    from deca_amd.kernels.rowwise_hip import build_rowwise

    op, M, N, dtype = wl["op"], wl["M"], wl["N"], wl["dtype"]
    kern = build_rowwise(_spec(wl))
    nbytes = rowwise_bytes(op, M, N)
    # Rotate over enough (x, y) pairs that the working set is several times the
    # Infinity Cache, so that every step streams from HBM.
    nsets = max(2, -(-4 * MALL_BYTES // nbytes))
    sets = []
    for i in range(nsets):
        inputs = make_inputs(op, M, N, dtype, seed=i, std=2.0 if op == "softmax" else 1.0)
        sets.append((*inputs, torch.empty_like(inputs[0])))
    # wall time per step, and kernel time from events around the same launches
    wall, t_rot, first = _timed_steps(kern, sets, steps, warmup)
    t_same = kern.time(sets[:1], steps)
    gbs = nbytes / wall / 1e9
    res = {
        "workload": wl["name"],
        "metric": f"{op} {dtype} [{M},{N}] effective HBM GB/s",
        "value": gbs,
        "unit": "GB/s",
        "ms_per_step": wall * 1e3,
        "dtype": "f32 math, %s I/O" % ("bf16" if dtype == "bfloat16" else "f16"),
        "config": str(wl["cfg"]),
        "roofline": {
            "bound": "hbm", "achieved": nbytes / t_rot / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": nbytes / t_rot / 1e9 / HBM_PEAK_GBS, "traffic": None,
            "kernel_us": t_rot * 1e6, "kernel_us_same_buffers": t_same * 1e6,
            "algorithmic_bytes": nbytes, "buffer_sets": nsets, "timed_launches": [first, steps],
        },
    }
    res["roofline"].update(_board(kern, sets))
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(wl)
    del sets
    torch.cuda.empty_cache()
    return res


def _timed_steps(kern, sets, steps, warmup):
    """(wall seconds per step, event seconds per launch, index of the first timed launch
    among the kernel object's launches) over the same `steps` back-to-back launches cycling
    through the argument sets: the host clock is read, with the device idle, on either side
    of the region, and two events are recorded on the launch stream (torch's current stream)
    directly before the first and after the last launch inside it (`deca_launch_between`), so
    the event time can never exceed the wall time."""
    import torch

    n = len(sets)
    # Untimed spin-up: the GPU drops to idle clocks while the host runs the CPU
    # baseline of the previous workload, and takes tens of milliseconds of load to
    # come back (the reference warms up by time as well, attn_bench.py:46-55).
    t_end = time.perf_counter() + SPIN_UP_SECONDS
    i = 0
    while time.perf_counter() < t_end:
        for _ in range(8):
            kern(*sets[i % n])
            i += 1
        torch.cuda.synchronize()
    for i in range(warmup):
        kern(*sets[i % n])
    packed = kern.pack(sets)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()  # (an event is created at its first record: not inside the timed region)
    stop.record()
    run = kern.batch_call(packed, steps, start, stop)
    torch.cuda.synchronize()
    first = kern.launches
    t0 = time.perf_counter()
    run()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return wall, start.elapsed_time(stop) * 1e-3 / steps, first


def run_gemm(wl, steps, warmup, with_cpu):
    import torch

    from deca_amd.kernels.gemm_bench import gemm_flops, make_inputs
    from deca_amd.kernels.gemm_hip import build_gemm_tc

    M, N, K = wl["M"], wl["N"], wl["K"]
    kern = build_gemm_tc(_spec(wl))
    tdt = torch.bfloat16 if wl["dtype"] == "bfloat16" else torch.float16
    short = "bf16" if wl["dtype"] == "bfloat16" else "f16"
    a, b = make_inputs(M, N, K, seed=0, dist="uniform", dtype=tdt)
    c = torch.empty(M, N, dtype=tdt, device="cuda")
    wall, t_k, first = _timed_steps(kern, [(a, b, c)], steps, warmup)
    flops = gemm_flops(M, N, K)
    board = _board(kern, [(a, b, c)])
    # the same kernel on the reference's operand distribution, N(0,1) (gemm_bench.py:26-31):
    # the board is power-limited and the rate follows the operand statistics
    a, b = make_inputs(M, N, K, seed=0, dist="normal", dtype=tdt)
    kern.time([(a, b, c)], max(5, steps // 2))
    t_n01 = kern.time([(a, b, c)], steps)
    res = {
        "workload": wl["name"],
        "metric": f"{'bf16' if short == 'bf16' else 'fp16'} GEMM {M}x{N}x{K} (fp32 accumulate) TFLOPS",
        "value": flops / wall / 1e12, "unit": "TFLOP/s", "ms_per_step": wall * 1e3,
        "dtype": f"{short} in/out, f32 accumulate", "config": str(wl["cfg"]),
        "roofline": {"bound": "mfma", "achieved": flops / t_k / 1e12, "peak": MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / t_k / 1e12 / MFMA_PEAK_TFLOPS,
                     "traffic": None, "kernel_us": t_k * 1e6, "algorithmic_flops": flops,
                     "timed_launches": [first, steps],
                     "achieved_normal_inputs": flops / t_n01 / 1e12},
    }
    res["roofline"].update(board)
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(wl)
    del a, b, c
    torch.cuda.empty_cache()
    return res


def run_fa(wl, steps, warmup, with_cpu):
    import torch

    from deca_amd.kernels.attn_bench import attn_flops, make_qkv
    from deca_amd.kernels.flash_attn_hip import build_flash_attn

    B, H, S, D, causal = wl["B"], wl["H"], wl["S"], wl["D"], wl["causal"]
    kern = build_flash_attn(_spec(wl))
    q, k, v = make_qkv(B, H, S, S, D, seed=0)
    o = torch.empty_like(q)
    wall, t_k, first = _timed_steps(kern, [(q, k, v, o)], steps, warmup)
    flops = attn_flops(B, H, S, S, D, causal)
    res = {
        "workload": wl["name"],
        "metric": f"FlashAttention fwd fp16 B{B} H{H} S{S} D{D}{' causal' if causal else ''} TFLOPS",
        "value": flops / wall / 1e12, "unit": "TFLOP/s", "ms_per_step": wall * 1e3,
        "dtype": "f16 in/out, f32 accumulate", "config": str(wl["cfg"]),
        "roofline": {"bound": "mfma", "achieved": flops / t_k / 1e12, "peak": MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / t_k / 1e12 / MFMA_PEAK_TFLOPS,
                     "traffic": None, "kernel_us": t_k * 1e6, "algorithmic_flops": flops,
                     "timed_launches": [first, steps]},
    }
    res["roofline"].update(_board(kern, [(q, k, v, o)]))
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(wl)
    del q, k, v, o
    torch.cuda.empty_cache()
    return res


def _measured_traffic(name, config):
    """HBM-side bytes per launch measured with rocprofv3 counters (see
    deca_amd/measured_traffic.json and profiles/).  The figure belongs to the
    kernel configuration it was measured on: None when nothing is recorded for
    the workload or the record is for another configuration than the timed one."""
    path = os.path.join(ROOT, "deca_amd", "measured_traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        entry = json.load(f).get("workloads", {}).get(name)
    if not entry or entry.get("config") != config:
        return None
    return entry["traffic_bytes"]


# The roofline fractions the task sets for the gated workloads (of 8 TB/s HBM
# bandwidth, or of 2.5 PFLOP/s dense fp16 MFMA).
TARGET_FRAC = {
    "rmsnorm_bf16_16384x4096": 0.80,
    "softmax_fp16_16384x4096": 0.80,
    "rmsnorm_fp16_8192x8192": 0.80,
    "gemm_fp16_8192": 0.70,
    "fa_fp16_b4h16s4096d128": 0.55,
}


def _compact(res):
    """What a reader needs to recompute one workload's roofline fraction:
    frac = work / (kernel_us * 1e-6) / (peak * 1e9 or 1e12)."""
    rf = res["roofline"]
    row = {
        "value": round(res["value"], 1), "unit": res["unit"],
        "ms_per_step": round(res["ms_per_step"], 5),
        "kernel_us": round(rf["kernel_us"], 2),
        "work": int(rf.get("algorithmic_bytes", rf.get("algorithmic_flops"))),
        "achieved": round(rf["achieved"], 1), "peak": rf["peak"], "frac": round(rf["frac"], 4),
        "traffic": rf["traffic"], "kernel_config": res["config"],
    }
    if "achieved_normal_inputs" in rf:
        row["achieved_n01"] = round(rf["achieved_normal_inputs"], 1)
    for key in ("sclk_mhz", "socket_w"):
        if key in rf:
            row[key] = rf[key]
    target = TARGET_FRAC.get(res["workload"])
    if target is not None:
        row["target_frac"] = target
        row["target_met"] = bool(rf["frac"] >= target)
    return row


def _compact_cpu(cb):
    """The CPU baseline of a workload without its description."""
    return {"value": float("%.4g" % cb["value"]), "unit": cb["unit"], "cores": cb["cores"],
            "seconds": round(cb["seconds"], 4)}


# The record has to fit the tail of standard output a harness keeps of a run.
MAX_RECORD_BYTES = 8192


def build_record(results, steps, warmup):
    """The one JSON object of a run.  `results[0]` is the headline workload; the
    others appear in compact form under roofline.all / cpu_baseline.all.  The
    full per-workload records go to a side file, not into the line."""
    head = results[0]
    out = {
        "metric": head["metric"],
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": head["workload"], "kernel_config": head["config"]},
        "roofline": dict(head["roofline"], all={r["workload"]: _compact(r) for r in results}),
    }
    if "cpu_baseline" in head:
        cb = head["cpu_baseline"]
        out["cpu_baseline"] = {
            "value": cb["value"], "unit": cb["unit"], "cores": cb["cores"], "kind": cb["kind"],
            "sample": cb["sample"], "seconds": cb["seconds"],
            "all": {r["workload"]: _compact_cpu(r["cpu_baseline"])
                    for r in results if "cpu_baseline" in r}}
    gated = {r["workload"]: _compact(r) for r in results if r["workload"] in TARGET_FRAC}
    out["config"]["targets_met"] = sorted(n for n, c in gated.items() if c["target_met"])
    out["config"]["targets_missed"] = {n: {"frac": c["frac"], "target": c["target_frac"]}
                                       for n, c in gated.items() if not c["target_met"]}
    return out


def print_table(results, file):
    """One line per workload."""
    print(f"[bench] {'workload':32s} {'value':>10s} {'unit':8s} {'kernel us':>10s} {'frac':>6s} "
          f"{'target':>6s}  config", file=file)
    for r in results:
        c = _compact(r)
        tgt = f"{c['target_frac']:.2f}" if "target_frac" in c else "  -"
        print(f"[bench] {r['workload']:32s} {c['value']:10.1f} {c['unit']:8s} {c['kernel_us']:10.2f} "
              f"{c['frac']:6.3f} {tgt:>6s}  {c['kernel_config']}", file=file)
    file.flush()


def run(wl, steps, warmup, with_cpu=True):
    t0 = time.perf_counter()
    print(f"[bench] {wl['name']} ...", file=sys.stderr, flush=True)
    res = {"rowwise": run_rowwise, "gemm": run_gemm, "fa": run_fa}[wl["kind"]](
        wl, steps, warmup, with_cpu)
    res["roofline"]["traffic"] = _measured_traffic(wl["name"], res["config"])
    print(f"[bench] {wl['name']}: {res['value']:.1f} {res['unit']} "
          f"({100 * res['roofline']['frac']:.1f}% of peak) in {time.perf_counter() - t0:.1f} s",
          file=sys.stderr, flush=True)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD)
    ap.add_argument("--kernel-config", default=None, metavar="TEXT",
                    help="time this kernel configuration (in the form the records print) for "
                         "--workload instead of its stored winner; implies --no-extra")
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--power", type=int, default=0, metavar="SECONDS",
                    help="after timing a workload, sample shader clock and socket power once a "
                         "second for this long while its kernel repeats (roofline.sclk_mhz / socket_w)")
    ap.add_argument("--full-out", default=os.path.join(ROOT, "bench_full.json"),
                    metavar="PATH", help="file for the full per-workload records ('' for none)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every workload is a single-device kernel "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the kernels have no host path)", file=sys.stderr)
        sys.exit(1)
    global POWER_SECONDS
    POWER_SECONDS = args.power
    wls = workloads()
    if args.kernel_config:
        from deca_amd import tuned

        wl = wls[args.workload]
        op = {"gemm": "GEMM", "fa": "flash_attn"}.get(wl["kind"]) or wl["op"]
        wl["cfg"] = tuned.parse_config(op, args.kernel_config)
        args.no_extra = True
    results = [run(wls[args.workload], args.steps, args.warmup, not args.no_cpu)]
    if not args.no_extra:
        # the other benchmark configurations, with fewer steps each so that the
        # default run stays within a few minutes
        k = max(5, min(args.steps, 30))
        results += [run(wl, k, min(args.warmup, 5), not args.no_cpu)
                    for name, wl in wls.items() if name != args.workload]
    out = build_record(results, args.steps, args.warmup)
    if args.full_out:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.full_out)), exist_ok=True)
            with open(args.full_out, "w") as f:
                json.dump(dict(out, results=results), f, indent=1)
        except OSError as e:
            print(f"[bench] full record not written: {e}", file=sys.stderr)
    # The table first, the record last: nothing follows the JSON line.
    print_table(results, sys.stderr)
    line = json.dumps(out, separators=(",", ":"))
    if len(line) > MAX_RECORD_BYTES:
        print(f"[bench] record is {len(line)} bytes (limit {MAX_RECORD_BYTES})", file=sys.stderr)
    sys.stderr.flush()
    print(line, flush=True)


if __name__ == "__main__":
    main()
