"""
Shared shapes / references for the row-wise operators (Softmax, RMSNorm).

Both operators are memory bound, so they are reported in GB/s of effective
DRAM traffic (read x [+ weight] + write y).  Counterpart of the reference's
src/kernels/rowwise_bench.py.
"""

from deca_amd.kernels.attn_bench import bench_cuda, bench_interleaved  # noqa: F401  (re-exported)

ROWWISE_OPS = ("softmax", "rmsnorm")
HIDDEN_SIZES = [1024, 2048, 4096, 8192]
HIDDEN_ROWS = [4096, 16384, 65536]
VOCAB_SIZES = [32000, 128256]
VOCAB_ROWS = [1024, 4096, 8192]
RMSNORM_EPS = 1e-6

DTYPE_ALIASES = {"fp16": "float16", "bf16": "bfloat16", "float16": "float16", "bfloat16": "bfloat16"}


def torch_dtype(dtype: str):
    import torch

    return {"float16": torch.float16, "bfloat16": torch.bfloat16}[canonical_dtype(dtype)]


def canonical_dtype(dtype: str) -> str:
    return DTYPE_ALIASES[dtype]


def standard_shapes(op: str):
    """Returns a list of (M, N)."""
    shapes = [(M, N) for N in HIDDEN_SIZES for M in HIDDEN_ROWS]
    if op == "softmax":
        shapes += [(M, N) for N in VOCAB_SIZES for M in VOCAB_ROWS]
    return shapes


def rowwise_bytes(op: str, M: int, N: int, type_size: int = 2) -> int:
    nbytes = 2 * M * N * type_size
    return nbytes + N * type_size if op == "rmsnorm" else nbytes


def make_inputs(op: str, M: int, N: int, dtype: str, seed: int = 0, device: str = "cuda",
                std: float = 1.0):
    """Returns the kernel inputs: (x,) for softmax, (x, w) for RMSNorm, with
    x ~ N(0, std^2) and w = 1 + 0.1 * randn (reference: rowwise_bench.py:42-50).
    The generator lives on `device`; "cpu" gives bits that are the same on
    every machine (see `make_inputs_cpu`)."""
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    tdt = torch_dtype(dtype)
    if device == "cpu":
        x = torch.randn(M, N, generator=g)
        if std != 1.0:
            x *= std
        x = x.to(tdt)
    else:
        x = torch.randn(M, N, device=device, dtype=tdt, generator=g)
        if std != 1.0:
            x = (x.float() * std).to(tdt)
    if op == "softmax":
        return (x,)
    w = (1.0 + 0.1 * torch.randn(N, device=device, generator=g)).to(tdt)
    return (x, w)


def make_inputs_cpu(op: str, M: int, N: int, dtype: str, seed: int = 0, std: float = 1.0):
    """Host tensors from a CPU generator: what the parity tests feed to both
    the checker and (after a copy) the device."""
    return make_inputs(op, M, N, dtype, seed, "cpu", std)


def torch_ref(op: str, inputs, eps: float = RMSNORM_EPS):
    """Eager torch baseline (also the correctness reference while tuning)."""
    import torch
    import torch.nn.functional as F

    if op == "softmax":
        (x,) = inputs
        return torch.softmax(x, dim=-1)
    x, w = inputs
    return F.rms_norm(x, (x.shape[-1],), w, eps=eps)


def bench_torch(op: str, M: int, N: int, dtype: str):
    """Returns (seconds, GB/s) of the eager torch operator on the device."""
    inputs = make_inputs(op, M, N, dtype)
    t = bench_cuda(lambda: torch_ref(op, inputs))
    return t, rowwise_bytes(op, M, N) / t / 1e9
