#!/usr/bin/env python3
"""Benchmark of the tuned kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra]

A step is one launch of the workload's kernel over one batch of synthetic
input already resident in HBM.  Prints ONE JSON line: the headline workload's
throughput (`value`), its roofline fraction measured with HIP events on the
launch stream, the torch-CPU baseline timed on this box's host cores, and --
unless --no-extra -- the same figures for the other benchmark configurations
under "results".
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


def _tuned():
    with open(os.path.join(ROOT, "deca_amd", "tuned_configs.json")) as f:
        return json.load(f)


def _row_cfg(d):
    from deca_amd.kernels.rowwise_hip import RowConfig

    return RowConfig(**d)


# name -> description of the workload
def workloads():
    t = _tuned()
    w = {}
    for name, (op, M, N, dtype) in {
        "rmsnorm_bf16_16384x4096": ("rmsnorm", 16384, 4096, "bfloat16"),
        "softmax_fp16_16384x4096": ("softmax", 16384, 4096, "float16"),
        "rmsnorm_fp16_8192x8192": ("rmsnorm", 8192, 8192, "float16"),
    }.items():
        w[name] = {"kind": "rowwise", "op": op, "M": M, "N": N, "dtype": dtype,
                   "cfg": _row_cfg(t[name])}
    return w


DEFAULT_WORKLOAD = "rmsnorm_bf16_16384x4096"


def _spec(wl):
    from deca_amd.kernels.rowwise_hip import make_rowwise

    if wl["kind"] == "rowwise":
        return make_rowwise(wl["op"], wl["M"], wl["N"], wl["dtype"], wl["cfg"], 1e-6)
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

    return ob.time_cpu(wl, torch.get_num_threads())


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
    for i in range(warmup):
        kern(*sets[i % nsets])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        kern(*sets[i % nsets])
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    # kernel time: HIP events around the same launches on the launch stream
    t_rot = kern.time(sets, steps)
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
            "algorithmic_bytes": nbytes, "buffer_sets": nsets,
        },
    }
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(wl)
    del sets
    torch.cuda.empty_cache()
    return res


def run(wl, steps, warmup, with_cpu=True):
    if wl["kind"] == "rowwise":
        return run_rowwise(wl, steps, warmup, with_cpu)
    raise ValueError(wl["kind"])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD)
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every workload is a single-device kernel "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the kernels have no host path)", file=sys.stderr)
        sys.exit(1)
    wls = workloads()
    for k, v in wls.items():
        v["name"] = k
    head = run(wls[args.workload], args.steps, args.warmup, not args.no_cpu)
    out = {
        "metric": head["metric"],
        "value": head["value"],
        "unit": head["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": args.workload, "kernel_config": head["config"]},
        "roofline": head["roofline"],
    }
    if "cpu_baseline" in head:
        out["cpu_baseline"] = head["cpu_baseline"]
    if not args.no_extra:
        out["results"] = [head] + [
            run(wl, args.steps, args.warmup, not args.no_cpu)
            for name, wl in wls.items() if name != args.workload
        ]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
