"""
Shared shapes / references for the FP16 MFMA GEMM (C = A @ B).

A[M, K], B[K, N] and C[M, N] are row-major float16; accumulation is fp32.
Counterpart of the reference's src/kernels/gemm_bench.py (its cuBLAS
fp16-accumulate wrapper, :47-85, has no equivalent: MFMA always accumulates
in fp32).
"""

from deca_amd.kernels.attn_bench import bench_cuda, bench_interleaved  # noqa: F401  (re-exported)

# Square GEMMs from 2K to 16K in steps of 2K.
SQUARE_SIZES = list(range(2048, 16384 + 1, 2048))


def standard_shapes():
    """Returns a list of (M, N, K)."""
    return [(n, n, n) for n in SQUARE_SIZES]


def gemm_flops(M: int, N: int, K: int) -> float:
    return 2.0 * M * N * K


def make_inputs(M: int, N: int, K: int, seed: int = 0, device: str = "cuda",
                dist: str = "normal", dtype=None):
    """Returns (a, b): unit-variance fp16 entries (reference:
    gemm_bench.py:26-31) or, with dist="uniform", entries ~ U(-1, 1)."""
    import torch

    dtype = dtype or torch.float16
    g = torch.Generator(device=device).manual_seed(seed)

    def draw(r, c):
        if dist == "uniform":
            return (2 * torch.rand(r, c, device=device, generator=g) - 1).to(dtype)
        if device == "cpu":
            return torch.randn(r, c, generator=g).to(dtype)
        return torch.randn(r, c, device=device, dtype=dtype, generator=g)

    return draw(M, K), draw(K, N)


def make_inputs_cpu(M: int, N: int, K: int, seed: int = 0, dist: str = "normal", dtype=None):
    """Host tensors from a CPU generator (identical bits on every machine)."""
    return make_inputs(M, N, K, seed, "cpu", dist, dtype)


def torch_ref(inputs):
    """torch (hipBLASLt / rocBLAS) baseline."""
    a, b = inputs
    return a @ b


def bench_torch(M: int, N: int, K: int):
    """Returns (seconds, TFLOPS) of torch.matmul on the device."""
    inputs = make_inputs(M, N, K)
    t = bench_cuda(lambda: torch_ref(inputs))
    return t, gemm_flops(M, N, K) / t / 1e12
