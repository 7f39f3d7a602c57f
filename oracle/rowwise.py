"""
numpy restatement of the reference's row-wise kernels.  Test infrastructure:
see the package docstring for who may import this.

Follows src/kernels/rowwise_tir.py:
  softmax, reg mode      :278-300   m2 = max(x) * log2e; e = exp2(x * log2e - m2);
                                    y = dtype(e * (1 / sum e))
  softmax, twopass mode  :301-338   per-lane online (max, sum) over `unroll`
                                    chunks per step, cross-lane combine
                                    sum_t s_t * exp2(m_t - m)
  rmsnorm                :339-389   r = rsqrt(sum(x^2) * (1 / N) + eps);
                                    y = dtype(f32(dtype(x * r)) * f32(w))
  neutral tail values    :35, :199-205  (-1e30 for max/exp, 0 for squares)
  traffic formula        src/kernels/rowwise_bench.py:37-39

Pinned by (tests/test_oracle_rowwise.py): torch.softmax and F.rms_norm on the
CPU (library routines), rows summing to 1, shift invariance, constant rows
-> 1/N, a row holding the fp16 maximum, all-ones RMSNorm -> 1/sqrt(1+eps),
scale invariance of RMSNorm, bf16 rounding against torch's own conversion, and
twopass == reg on the same rows.
"""

from __future__ import annotations

import numpy as np

LOG2E = np.float32(1.4426950408889634)
NEG_INF = np.float32(-1e30)


def round_to_dtype(a: np.ndarray, dtype: str) -> np.ndarray:
    """Round-to-nearest-even of fp32 values to `dtype`, returned as fp32."""
    a = np.asarray(a, dtype=np.float32)
    if dtype == "float16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16).astype(np.float32)
    if dtype == "bfloat16":
        bits = a.view(np.uint32).astype(np.uint64)
        lsb = (bits >> 16) & 1
        rounded = ((bits + 0x7FFF + lsb) >> 16) << 16
        out = (rounded & 0xFFFFFFFF).astype(np.uint32).view(np.float32)
        nan = np.isnan(a)
        if nan.any():
            out = np.where(nan, np.float32(np.nan), out)
        return out.reshape(a.shape)
    raise ValueError(dtype)


def softmax_reg(x: np.ndarray, dtype: str) -> np.ndarray:
    """x: [M, N] fp32 holding `dtype`-representable values.  Returns fp32
    holding the `dtype`-rounded result (rowwise_tir.py:278-300)."""
    x = np.asarray(x, dtype=np.float32)
    m2 = x.max(axis=-1, keepdims=True) * LOG2E
    e = np.exp2(x * LOG2E - m2, dtype=np.float32)
    inv = np.float32(1.0) / e.sum(axis=-1, keepdims=True, dtype=np.float32)
    return round_to_dtype(e * inv, dtype)


def softmax_twopass(x: np.ndarray, dtype: str, threads_per_row: int, vec: int,
                    unroll: int) -> np.ndarray:
    """Lane-by-lane restatement of the streaming softmax (rowwise_tir.py:301-338).
    Each of the `threads_per_row` lanes keeps a running (max, sum) over its
    chunks, `unroll` chunks per step; the row result combines the lanes."""
    x = np.asarray(x, dtype=np.float32)
    M, N = x.shape
    span = threads_per_row * vec
    chunks = -(-N // span)
    c_full = N // span
    n_loop = c_full // unroll
    groups = [list(range(g * unroll, (g + 1) * unroll)) for g in range(n_loop)]
    groups += [[c] for c in range(n_loop * unroll, chunks)]
    # pad the row with the neutral value so that tail lanes read -1e30
    pad = chunks * span - N
    xp = np.concatenate([x, np.full((M, pad), NEG_INF, np.float32)], axis=1)
    xp = xp.reshape(M, chunks, threads_per_row, vec)  # [row, chunk, lane, i]
    run_m = np.full((M, threads_per_row), NEG_INF, np.float32)
    run_s = np.zeros((M, threads_per_row), np.float32)
    for grp in groups:
        vals = xp[:, grp].transpose(0, 2, 1, 3).reshape(M, threads_per_row, -1) * LOG2E
        # the kernel scales only in-row values; out-of-row lanes stay at -1e30
        vals = np.where(xp[:, grp].transpose(0, 2, 1, 3).reshape(M, threads_per_row, -1) == NEG_INF,
                        NEG_INF, vals)
        new_m = np.maximum(run_m, vals.max(axis=-1))
        run_s = run_s * np.exp2(run_m - new_m, dtype=np.float32) + np.exp2(
            vals - new_m[..., None], dtype=np.float32
        ).sum(axis=-1, dtype=np.float32)
        run_m = new_m
    m2 = run_m.max(axis=-1, keepdims=True)
    tot = (run_s * np.exp2(run_m - m2, dtype=np.float32)).sum(axis=-1, keepdims=True,
                                                              dtype=np.float32)
    inv = np.float32(1.0) / tot
    e = np.exp2(x * LOG2E - m2, dtype=np.float32)
    return round_to_dtype(e * inv, dtype)


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float, dtype: str) -> np.ndarray:
    """x: [M, N], w: [N] fp32 holding `dtype` values (rowwise_tir.py:339-389).
    The normalised value is rounded to `dtype` before the weight multiply."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    N = x.shape[-1]
    ss = (x * x).sum(axis=-1, keepdims=True, dtype=np.float32)
    r = np.float32(1.0) / np.sqrt(ss * np.float32(1.0 / N) + np.float32(eps), dtype=np.float32)
    normed = round_to_dtype(x * r, dtype)
    return round_to_dtype(normed * w, dtype)


def rowwise_bytes(op: str, M: int, N: int, type_size: int = 2) -> int:
    """Algorithmic traffic: read x (+ w) and write y (rowwise_bench.py:37-39)."""
    n = 2 * M * N * type_size
    return n + N * type_size if op == "rmsnorm" else n


def to_f32(t) -> np.ndarray:
    """torch CPU tensor (fp16 / bf16 / fp32) -> fp32 numpy array."""
    return t.detach().to("cpu").float().numpy()
