"""CPU baseline timings for bench.py: torch's CPU operators on a bounded sample
of each workload, on this machine's host cores.  Test/measurement
infrastructure only -- nothing under deca_amd/ imports this."""

from __future__ import annotations

import time


def _median_time(fn, warmup=1, reps=3):
    for _ in range(warmup):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


def time_cpu(wl: dict, threads: int) -> dict:
    import os

    import torch
    import torch.nn.functional as F

    if wl["kind"] == "rowwise":
        op, M, N, dtype = wl["op"], wl["M"], wl["N"], wl["dtype"]
        tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float16
        g = torch.Generator().manual_seed(0)
        x = torch.randn(M, N, generator=g).to(tdt)
        if op == "softmax":
            fn = lambda: torch.softmax(x, -1)  # noqa: E731
            what = f"torch.softmax(x_cpu, -1), full [{M},{N}] {dtype} tensor"
        else:
            w = (1 + 0.1 * torch.randn(N, generator=g)).to(tdt)
            fn = lambda: F.rms_norm(x, (N,), w, eps=1e-6)  # noqa: E731
            what = f"F.rms_norm(x_cpu, ({N},), w, 1e-6), full [{M},{N}] {dtype} tensor"
        t = _median_time(fn)
        nbytes = 2 * M * N * 2 + (N * 2 if op == "rmsnorm" else 0)
        return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": what + ", 1 warm-up, median of 3", "seconds": t,
                "host_cpus": os.cpu_count()}
    raise ValueError(wl["kind"])
