"""
numpy restatement of the reference's GEMM arithmetic.  Test infrastructure:
see the package docstring for who may import this.

Follows src/kernels/gemm_tir.py: C[m, n] = fp16( sum_k fp32(A[m, k]) * fp32(B[k, n]) )
with fp32 products and accumulation (:280-290, fp32 accumulators :236-238) and
one round-to-nearest conversion at the end (:336-346); A [M, K], B [K, N],
C [M, N] row-major (:12, :150-152).  The accumulation order inside the
hardware differs from any fixed order, so the checker offers the fp32 matmul
(`gemm_f32`) and an fp64 one (`gemm_f64`) whose distance bounds the ordering
effect; the verification metric of src/operators/GEMMTC.py:51-63 and
src/RuntimeMod.py:210-225 is `excess`.

Pinned by (tests/test_oracle_gemm.py): a brute-force triple loop on small
sizes, identity and one-hot operands (transposition / layout), all-ones
operands (every entry equals K; exact in fp16 up to 2048), non-square shapes,
and an fp32-vs-fp16-accumulation discriminator (K = 16384, entries 0.01).
"""

from __future__ import annotations

import math

import numpy as np


def gemm_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """fp32 accumulate of fp16-valued inputs, un-rounded (the accuracy reference)."""
    return np.asarray(a, np.float32) @ np.asarray(b, np.float32)


def gemm_f64(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    return np.asarray(a, np.float64) @ np.asarray(b, np.float64)


def gemm_f16_out(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """What the kernel stores: the fp32 result rounded once to fp16 (as fp32 values)."""
    with np.errstate(over="ignore"):
        return gemm_f32(a, b).astype(np.float16).astype(np.float32)


def gemm_bf16_out(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """The bf16 variant (no counterpart in the reference, which is fp16 only):
    same fp32 accumulation, one round-to-nearest-even conversion to bf16."""
    from oracle.rowwise import round_to_dtype

    return round_to_dtype(gemm_f32(a, b), "bfloat16")


def gemm_loops(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Triple loop in fp32, k ascending (small sizes only)."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    M, K = a.shape
    N = b.shape[1]
    c = np.zeros((M, N), np.float32)
    for m in range(M):
        for n in range(N):
            acc = np.float32(0)
            for k in range(K):
                acc = np.float32(acc + a[m, k] * b[k, n])
            c[m, n] = acc
    return c


def tolerance(K: int):
    """(atol, rtol) of the reference's check (GEMMTC.py:51-63)."""
    return (1e-2 * math.sqrt(K / 1024), 2e-3)


def excess(c: np.ndarray, ref: np.ndarray, K: int) -> float:
    """max |c - ref| / (atol + rtol * |ref|); the reference accepts <= 1."""
    atol, rtol = tolerance(K)
    return float((np.abs(c - ref) / (atol + rtol * np.abs(ref))).max())


def max_rel_err(c: np.ndarray, ref: np.ndarray) -> float:
    """max |c - ref| / max |ref| (element-wise relative error is unbounded near zero)."""
    return float(np.abs(c - ref).max() / np.abs(ref).max())


def gemm_flops(M: int, N: int, K: int) -> float:
    return 2.0 * M * N * K
