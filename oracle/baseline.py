"""CPU baseline timings for bench.py: torch's CPU operators on a bounded sample
of each workload, on this machine's host cores.  Test/measurement
infrastructure only -- nothing under deca_amd/ imports this."""

from __future__ import annotations

import time


BUDGET_SECONDS = 4.0  # CPU time spent per workload on repetitions


def _median_time(fn, warmup=1, reps=3):
    """Median over at least `reps` runs, and as many more as fit BUDGET_SECONDS (<= 50).
    Returns (seconds, runs)."""
    for _ in range(warmup):
        fn()
    ts = []
    t_start = time.perf_counter()
    while len(ts) < reps or (len(ts) < 50 and time.perf_counter() - t_start < BUDGET_SECONDS):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], len(ts)


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
        t, runs = _median_time(fn)
        nbytes = 2 * M * N * 2 + (N * 2 if op == "rmsnorm" else 0)
        return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": what + f", 1 warm-up, median of {runs}", "seconds": t,
                "host_cpus": os.cpu_count()}
    if wl["kind"] == "gemm":
        # fp32 product of the fp16 inputs (also the accuracy reference).  torch's
        # CPU fp16 matmul has no vectorised path on every host (0.4 GFLOP/s on an
        # EPYC without AVX512-FP16), so it is only sampled on 8 rows.
        M, N, K = wl["M"], wl["N"], wl["K"]
        rows = min(M, max(64, int(4e11 / (2.0 * N * K))))  # ~0.4 TFLOP of work
        g = torch.Generator().manual_seed(0)
        tdt = torch.bfloat16 if wl.get("dtype") == "bfloat16" else torch.float16
        a = (2 * torch.rand(rows, K, generator=g) - 1).to(tdt)
        b = (2 * torch.rand(K, N, generator=g) - 1).to(tdt)
        af, bf = a.float(), b.float()
        t32, runs = _median_time(lambda: af @ bf, warmup=1, reps=3)
        small, b_cols = a[:8].contiguous(), b[:, :512].contiguous()
        t0 = time.perf_counter()
        small @ b_cols
        t16 = time.perf_counter() - t0
        flops = 2.0 * rows * N * K
        return {"value": flops / t32 / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"torch a_cpu.float() @ b_cpu.float() on the first {rows} of {M} rows "
                          f"of A (all of B), 1 warm-up, median of {runs}",
                "seconds": t32, "native_matmul_value": 2.0 * 8 * 512 * K / t16 / 1e12,
                "native_matmul_sample": f"a_cpu[:8] @ b_cpu[:, :512] in {wl.get('dtype', 'float16')}, single run",
                "host_cpus": os.cpu_count()}
    if wl["kind"] == "fa":
        B, H, S, D, causal = wl["B"], wl["H"], wl["S"], wl["D"], wl["causal"]
        heads = 2
        g = torch.Generator().manual_seed(0)
        q, k, v = (torch.randn(1, heads, S, D, generator=g).half() for _ in range(3))
        scale = D ** -0.5

        def math_attn():
            s = (q.float() @ k.float().transpose(-1, -2)) * scale
            if causal:
                s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
            return torch.softmax(s, -1) @ v.float()

        t, runs = _median_time(math_attn, warmup=1, reps=3)
        flops = 4.0 * heads * S * S * D / (2 if causal else 1)
        return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"fp32 softmax(scale QK^T + mask) V with torch on the CPU for {heads} of "
                          f"{B * H} (batch, head) slices, 1 warm-up, median of {runs}",
                "seconds": t, "host_cpus": os.cpu_count()}
    raise ValueError(wl["kind"])
