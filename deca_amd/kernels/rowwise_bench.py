"""
Shapes, traffic formula, inputs and torch references of the row-wise operators
(Softmax, RMSNorm).  Both are memory bound and are reported in GB/s of
effective DRAM traffic: read x (+ weight) and write y.  Counterpart of the
reference's src/kernels/rowwise_bench.py (same public names).
"""

from deca_amd.kernels.attn_bench import bench_cuda, bench_interleaved  # noqa: F401  (re-exported)

ROWWISE_OPS = ("softmax", "rmsnorm")
RMSNORM_EPS = 1e-6
# benchmark grid of the reference (rowwise_bench.py:15-18): transformer hidden
# sizes at three token counts, plus two vocabulary sizes for softmax
HIDDEN_SIZES = [1024, 2048, 4096, 8192]
HIDDEN_ROWS = [4096, 16384, 65536]
VOCAB_SIZES = [32000, 128256]
VOCAB_ROWS = [1024, 4096, 8192]
DTYPE_ALIASES = {"fp16": "float16", "float16": "float16", "bf16": "bfloat16", "bfloat16": "bfloat16"}


def canonical_dtype(dtype: str) -> str:
    return DTYPE_ALIASES[dtype]


def torch_dtype(dtype: str):
    import torch

    return getattr(torch, canonical_dtype(dtype))


def standard_shapes(op: str):
    """[(M, N)] of the sweep for `op`."""
    grid = [(M, N) for N in HIDDEN_SIZES for M in HIDDEN_ROWS]
    if op == "softmax":
        grid.extend((M, N) for N in VOCAB_SIZES for M in VOCAB_ROWS)
    return grid


def rowwise_bytes(op: str, M: int, N: int, type_size: int = 2) -> int:
    """x read once and y written once, plus the weight vector of RMSNorm."""
    return (2 * M * N + (N if op == "rmsnorm" else 0)) * type_size


def make_inputs(op: str, M: int, N: int, dtype: str, seed: int = 0, device: str = "cuda",
                std: float = 1.0):
    """(x,) for softmax, (x, w) for RMSNorm: x ~ N(0, std^2), w = 1 + 0.1 * randn
    (reference: rowwise_bench.py:42-50).  The generator lives on `device`; "cpu"
    gives bits that are identical on every machine (see `make_inputs_cpu`)."""
    import torch

    gen = torch.Generator(device=device).manual_seed(seed)
    tdt = torch_dtype(dtype)
    on_host = device == "cpu"
    x = torch.randn(M, N, device=device, generator=gen, dtype=torch.float32 if on_host else tdt)
    if std != 1.0:
        x = x.float() * std
    x = x.to(tdt)
    if op == "softmax":
        return (x,)
    w = torch.randn(N, device=device, generator=gen).mul_(0.1).add_(1.0).to(tdt)
    return (x, w)


def make_inputs_cpu(op: str, M: int, N: int, dtype: str, seed: int = 0, std: float = 1.0):
    """Host tensors from a CPU generator: what the parity tests feed to both the
    checker and (after a copy) the device."""
    return make_inputs(op, M, N, dtype, seed, "cpu", std)


def rotating_sets(inputs, out, cache_bytes: int, factor: int = 4):
    """Copies of (inputs..., out) whose total size is `factor` times the
    last-level cache, to be cycled through while timing a memory-bound kernel.

    The reference times every kernel on one set of buffers
    (attn_bench.py:46-70).  On MI355X one [16384, 4096] fp16 input/output pair
    is 268 MB next to a 256 MiB Infinity Cache, so a single set is partly served
    from that cache and over-states the HBM rate; rotating sets larger than the
    cache makes every launch stream from HBM."""
    per_set = sum(t.numel() * t.element_size() for t in (*inputs, out))
    n = max(1, -(-factor * cache_bytes // per_set))
    sets = [(*inputs, out)]
    for _ in range(n - 1):
        sets.append((*(t.clone() for t in inputs), out.clone()))
    return sets


def cycle(fn, sets):
    """A zero-argument callable that calls `fn(*sets[i])` with i advancing on every call."""
    state = {"i": 0}

    def call():
        args = sets[state["i"] % len(sets)]
        state["i"] += 1
        return fn(*args)

    return call


def torch_ref(op: str, inputs, eps: float = RMSNORM_EPS):
    """Eager torch operator: the baseline and the correctness reference while tuning."""
    import torch
    import torch.nn.functional as F

    x = inputs[0]
    if op == "softmax":
        return torch.softmax(x, dim=-1)
    return F.rms_norm(x, (x.shape[-1],), inputs[1], eps=eps)


def bench_torch(op: str, M: int, N: int, dtype: str):
    """(seconds, GB/s) of the eager torch operator on the device."""
    inputs = make_inputs(op, M, N, dtype)
    seconds = bench_cuda(lambda: torch_ref(op, inputs))
    return seconds, rowwise_bytes(op, M, N) / seconds / 1e9
