"""
Shared timing / reference helpers (the attention benchmarks own the event
harness that every operator reuses, as in the reference's
src/kernels/attn_bench.py).

Inputs are drawn from a CPU `torch.Generator` and copied to the device, so the
host-side checker and the GPU see identical bits on any machine (the reference
seeds a CUDA generator, attn_bench.py:73-78, whose stream is device specific).
"""

import math
import time
from typing import Callable

# FlashAttention-2 paper setup: hidden = 2048, batch * seqlen = 16k.
FA_SEQLENS = [512, 1024, 2048, 4096, 8192, 16384]
FA_HEADDIM_HEADS = [(64, 32), (128, 16)]


def standard_shapes():
    """Returns a list of (B, H, S, D)."""
    shapes = []
    for D, H in FA_HEADDIM_HEADS:
        for S in FA_SEQLENS:
            shapes.append((16384 // S, H, S, D))
    return shapes


def attn_flops(B: int, H: int, S_q: int, S_kv: int, D: int, causal: bool = False) -> float:
    flops = 4.0 * B * H * S_q * S_kv * D
    return flops / 2 if causal else flops


def bench_cuda(
    fn: Callable[[], None],
    warmup_s: float = 0.3,
    measure_s: float = 0.3,
    min_iters: int = 20,
) -> float:
    """Median time of `fn` in seconds, measured with one event pair per call
    on torch's current stream (which is the stream the kernels launch on).

    Warm-up and measurement are time based, as in the reference
    (attn_bench.py:35-70): short warm-ups leave the GPU at a lower clock.
    """
    import torch

    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < warmup_s:
        fn()
        torch.cuda.synchronize()
    probe_start = torch.cuda.Event(enable_timing=True)
    probe_end = torch.cuda.Event(enable_timing=True)
    probe_start.record()
    fn()
    probe_end.record()
    probe_end.synchronize()
    per_call = max(probe_start.elapsed_time(probe_end) / 1e3, 1e-6)
    iters = max(min_iters, int(measure_s / per_call))
    times = []
    for _ in range(iters):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end) / 1e3)
    times.sort()
    return times[len(times) // 2]


def bench_interleaved(fns: dict, rounds: int = 3) -> dict:
    """Times several callables alternately; returns the median per name (seconds)."""
    samples = {name: [] for name in fns}
    for _ in range(rounds):
        for name, fn in fns.items():
            samples[name].append(bench_cuda(fn))
    return {name: sorted(ts)[len(ts) // 2] for name, ts in samples.items()}


def make_qkv(B: int, H: int, S_q: int, S_kv: int, D: int, dtype=None, seed: int = 0,
             device: str = "cuda"):
    """q, k, v ~ N(0, 1) in [B, H, S, D] (reference: attn_bench.py:73-78)."""
    import torch

    dtype = dtype or torch.float16
    g = torch.Generator(device=device).manual_seed(seed)

    def draw(S):
        if device == "cpu":
            return torch.randn(B, H, S, D, generator=g).to(dtype)
        return torch.randn(B, H, S, D, device=device, dtype=dtype, generator=g)

    return draw(S_q), draw(S_kv), draw(S_kv)


def make_qkv_cpu(B: int, H: int, S_q: int, S_kv: int, D: int, dtype=None, seed: int = 0):
    """Host tensors from a CPU generator (identical bits on every machine)."""
    return make_qkv(B, H, S_q, S_kv, D, dtype, seed, "cpu")


def sdpa_flash(q, k, v, causal: bool = False, scale: float | None = None):
    """torch's fused attention on the device (the baseline the tuner reports
    against; reference: attn_bench.py:81-83)."""
    import torch.nn.functional as F

    return F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=scale)


def math_attention(q, k, v, causal: bool = False, scale: float | None = None):
    """fp32 softmax(scale * Q K^T + mask) V, head by head (accuracy reference
    of the attention kernel; works on CPU and device tensors)."""
    import torch

    B, H, S_q, D = q.shape
    S_kv = k.shape[2]
    scale = default_scale(D) if scale is None else scale
    out = torch.empty(B, H, S_q, D, dtype=torch.float32, device=q.device)
    mask = None
    if causal:
        mask = torch.ones(S_q, S_kv, dtype=torch.bool, device=q.device).tril()
    for b in range(B):
        for h in range(H):
            s = (q[b, h].float() @ k[b, h].float().T) * scale
            if mask is not None:
                s = s.masked_fill(~mask, float("-inf"))
            out[b, h] = torch.softmax(s, dim=-1) @ v[b, h].float()
    return out


def bench_sdpa_flash(B, H, S_q, S_kv, D, causal=False, dtype=None):
    """Returns (seconds, TFLOPS) of torch SDPA on the device."""
    q, k, v = make_qkv(B, H, S_q, S_kv, D, dtype)
    t = bench_cuda(lambda: sdpa_flash(q, k, v, causal))
    return t, attn_flops(B, H, S_q, S_kv, D, causal) / t / 1e12


def default_scale(D: int) -> float:
    return 1.0 / math.sqrt(D)
