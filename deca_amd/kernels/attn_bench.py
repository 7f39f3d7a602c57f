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

# Sweep grid of the FlashAttention-2 paper, as the reference uses it
# (attn_bench.py:14-27): 16k tokens per batch at a hidden size of 2048, i.e.
# head_dim x heads = 2048 and batch x seqlen = 16384.
FA_TOKENS = 16384
FA_HIDDEN = 2048
FA_SEQLENS = [512, 1024, 2048, 4096, 8192, 16384]
FA_HEADDIM_HEADS = [(D, FA_HIDDEN // D) for D in (64, 128)]


def standard_shapes():
    """The sweep grid as (B, H, S, D) tuples, head dims outermost."""
    return [(FA_TOKENS // S, H, S, D) for D, H in FA_HEADDIM_HEADS for S in FA_SEQLENS]


def attn_flops(B: int, H: int, S_q: int, S_kv: int, D: int, causal: bool = False) -> float:
    """Two S_q x S_kv x D products per head, 2 FLOPs per multiply-add; a causal
    mask leaves half of the score matrix (reference: attn_bench.py:30-32)."""
    products = 2.0 * (B * H) * S_q * S_kv * D
    return products if causal else 2.0 * products


class _EventTimer:
    """Times single calls on torch's current stream (the stream every kernel of
    this package is launched on) with a reusable pool of event pairs."""

    def __init__(self, pairs: int = 64):
        import torch

        self._torch = torch
        self._pool = [self._pair() for _ in range(pairs)]

    def _pair(self):
        ev = self._torch.cuda.Event
        return ev(enable_timing=True), ev(enable_timing=True)

    def one(self, fn, slot: int = 0) -> float:
        """Seconds of one call that starts on an idle stream."""
        while slot >= len(self._pool):
            self._pool.append(self._pair())
        first, last = self._pool[slot]
        first.record()
        fn()
        last.record()
        last.synchronize()
        return first.elapsed_time(last) * 1e-3

    def spin(self, fn, seconds: float) -> float:
        """Keeps calling `fn` for `seconds` of wall-clock time so that the clocks
        settle; returns the duration of the last call."""
        deadline = time.perf_counter() + seconds
        last = self.one(fn)
        while time.perf_counter() < deadline:
            last = self.one(fn)
        return last

    def samples(self, fn, count: int) -> list:
        return [self.one(fn, i % len(self._pool)) for i in range(count)]


_timer = None


def _event_timer() -> _EventTimer:
    global _timer
    if _timer is None:
        _timer = _EventTimer()
    return _timer


def _median(values) -> float:
    ordered = sorted(values)
    return ordered[len(ordered) // 2]


def bench_cuda(fn, warmup_s: float = 0.3, measure_s: float = 0.3, min_iters: int = 20) -> float:
    """Median seconds per call of `fn`.

    Same measurement as the reference's helper of this name
    (attn_bench.py:35-70): a warm-up that lasts `warmup_s` of wall-clock time
    (a fixed number of calls leaves the GPU at a low clock for short kernels),
    then about `measure_s` worth of calls and never fewer than `min_iters`, each
    bracketed by its own event pair and followed by a synchronisation; the
    result is the median of those single-call times.
    """
    timer = _event_timer()
    settled = max(timer.spin(fn, warmup_s), 1e-6)
    count = max(int(min_iters), int(measure_s / settled))
    return _median(timer.samples(fn, count))


def bench_interleaved(fns: dict, rounds: int = 3) -> dict:
    """Median of `rounds` bench_cuda results per entry of `fns`, the entries
    taking turns in every round so that drift (clocks, temperature) hits all of
    them alike (reference: attn_bench.py:94-100)."""
    per_name = {name: [] for name in fns}
    for _ in range(rounds):
        for name in per_name:
            per_name[name].append(bench_cuda(fns[name]))
    return {name: _median(seen) for name, seen in per_name.items()}


TIMINGS = ("events", "back_to_back")


def batch_timer(fn):
    """`timed(n)` -> average seconds of n back-to-back calls of `fn` on torch's current
    stream, between one pair of events.  A kernel loaded by this package brings its own
    (`LoadedKernel.time`, whose launches stay inside the launcher library); this is for
    callables that go through torch."""
    import torch

    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(n: int) -> float:
        first.record()
        for _ in range(n):
            fn()
        last.record()
        last.synchronize()
        return first.elapsed_time(last) * 1e-3 / n

    return timed


def bench_back_to_back(timed, warmup_s: float = 0.3, measure_s: float = 0.3,
                       min_iters: int = 20, batches: int = 3) -> float:
    """Seconds per call from batches of calls issued back to back (`timed(n)`, see
    `batch_timer`): a time-based warm-up as in `bench_cuda`, then `batches` batches that
    together last about `measure_s`; the median batch.  Unlike the one-call-per-event-pair
    timing of `bench_cuda` (the reference's, attn_bench.py:35-70) the GPU never idles
    between calls, which is how a kernel runs inside a model and what bench.py times: on a
    power-limited board the two rank near-equal candidates differently."""
    deadline = time.perf_counter() + warmup_s
    settled = timed(4)
    while time.perf_counter() < deadline:
        settled = timed(8)
    count = max(int(min_iters), int(measure_s / max(settled, 1e-7) / batches))
    return _median([timed(count) for _ in range(batches)])


def bench_interleaved_batches(timers: dict, rounds: int = 3) -> dict:
    """`bench_interleaved` for batch timers (name -> `timed(n)`)."""
    per_name = {name: [] for name in timers}
    for _ in range(rounds):
        for name in per_name:
            per_name[name].append(bench_back_to_back(timers[name]))
    return {name: _median(seen) for name, seen in per_name.items()}


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


# Which torch attention back end `sdpa_flash` ran last ("flash" when the pin below
# held, "default" when torch chose); drivers print it beside the ratio column.
SDPA_BACKEND = "flash"


def sdpa_flash(q, k, v, causal: bool = False, scale: float | None = None):
    """torch's fused attention restricted to its flash back end, the baseline the
    tuner reports against (reference: attn_bench.py:81-83).  Where this torch
    build has no flash kernel for the inputs, torch picks the back end and
    `SDPA_BACKEND` says so."""
    global SDPA_BACKEND
    import torch.nn.functional as F

    if SDPA_BACKEND == "flash":
        try:
            from torch.nn.attention import SDPBackend, sdpa_kernel

            with sdpa_kernel(SDPBackend.FLASH_ATTENTION):
                return F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=scale)
        except (ImportError, RuntimeError):
            SDPA_BACKEND = "default"
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
