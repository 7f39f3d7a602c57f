"""
numpy restatement of the reference's FlashAttention forward arithmetic.  Test
infrastructure: see the package docstring for who may import this.

Follows src/kernels/flash_attn_tir.py:
  layout            :11, :139-142   Q, K, V, O contiguous [B, H, S, D] fp16
  causal mask       :93, :379-400   key j visible to query i iff j <= i; the
                                    masked score is -1e30
  online softmax    :403-438        per KV tile of Bc rows: m' = max(m, rowmax S);
                                    alpha = exp2((m - m') * sl2);
                                    p = exp2(S * sl2 - m' * sl2), sl2 = scale * log2e;
                                    l = l * alpha + sum p (fp32 p); P = fp16(p)
  second product    :441            O = O * alpha + P V  (fp16 P, fp32 accumulate)
  normalisation     :444-458        O / l rounded to fp16
  flop count        src/kernels/attn_bench.py:30-32

`attention_f32` is the plain fp32 softmax(scale * Q K^T + mask) V (the accuracy
reference); `flash_blockwise` follows the tiled recurrence above, including
the fp16 rounding of P.

Pinned by (tests/test_oracle_attn.py): torch's softmax-matmul composite on the
CPU, constant V -> O equals that constant, K = 0 -> uniform attention (O = mean
of V; causal: prefix mean, which pins the mask direction), the first causal row
attends to key 0 only, single-tile == multi-tile (pins the online rescale),
S_q != S_kv, and blockwise == plain within the fp16 rounding of P.
"""

from __future__ import annotations

import math

import numpy as np

LOG2E = 1.4426950408889634
NEG_INF = np.float32(-1e30)


def default_scale(D: int) -> float:
    return 1.0 / math.sqrt(D)


def attention_f32(q, k, v, scale=None, causal=False) -> np.ndarray:
    """[B, H, S_q, D] fp32 result (not rounded)."""
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    v = np.asarray(v, np.float32)
    B, H, S_q, D = q.shape
    S_kv = k.shape[2]
    scale = default_scale(D) if scale is None else scale
    out = np.empty((B, H, S_q, D), np.float32)
    mask = None
    if causal:
        mask = np.arange(S_kv)[None, :] > np.arange(S_q)[:, None]
    for b in range(B):
        for h in range(H):
            s = (q[b, h] @ k[b, h].T) * np.float32(scale)
            if mask is not None:
                s = np.where(mask, -np.inf, s)
            s = s - s.max(axis=-1, keepdims=True)
            p = np.exp(s, dtype=np.float32)
            out[b, h] = (p @ v[b, h]) / p.sum(axis=-1, keepdims=True, dtype=np.float32)
    return out


def flash_blockwise(q, k, v, scale=None, causal=False, Br=128, Bc=64, lazy_tau=0.0,
                    max_every=1, trust_bound=None, wave_rows=32, key_groups=(8, 4),
                    sum_p16=False, stats=None) -> np.ndarray:
    """The tiled online-softmax recurrence; returns fp32 values rounded to fp16.

    `lazy_tau` = 0 is the reference's update m' = max(m, rowmax S)
    (flash_attn_tir.py:419-428).  With `lazy_tau` > 0 the running max only
    follows a tile's max that lies more than 2^lazy_tau above it (in units of
    the exponent, (m' - m) * sl2): the HIP kernel's variant, which leaves O / l
    the same quotient with p <= 2^lazy_tau.  `max_every` > 1 looks at a tile's
    max only in every `max_every`-th tile (a variant that was considered for the
    kernel and is NOT safe: nothing bounds p in the tiles between, see
    tests/test_oracle_attn.py).

    `trust_bound` (the kernel's `FAConfig.trust`, bound 2^15): every tile but the first (and,
    under the causal mask, but those that reach the diagonal for a wave) has its exponentials
    taken against the running max as it stands, without its own max.  The p of a lane are
    bounded by their sum, so a wave (`wave_rows` query rows) accepts the tile while no lane's
    sum exceeds the bound -- a lane holds the keys k of the tile with
    (k % key_groups[0]) // key_groups[1] == its group: (8, 4) for 32x32x16 tiles; `None` is one
    group, the sum over the whole tile -- and otherwise does the tile again with its max (lazy
    rule).  The kernel's plain loops on 16x16x32 tiles take these sums on the matrix pipe: over the whole
    tile (`key_groups=None`) and of the fp16 P that the second product sees (`sum_p16`),
    which is then also what l accumulates.  `stats`, a dict, receives the number of
    (wave, tile) pairs taken on trust and of those done again."""
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    v = np.asarray(v, np.float32)
    B, H, S_q, D = q.shape
    S_kv = k.shape[2]
    scale = default_scale(D) if scale is None else scale
    sl2 = np.float32(scale * LOG2E)
    out = np.empty((B, H, S_q, D), np.float32)
    for b in range(B):
        for h in range(H):
            for q0 in range(0, S_q, Br):
                qt = q[b, h, q0:q0 + Br]
                rows = np.arange(q0, q0 + qt.shape[0])
                m = np.full(qt.shape[0], NEG_INF, np.float32)
                l = np.zeros(qt.shape[0], np.float32)
                o = np.zeros((qt.shape[0], D), np.float32)
                kv_end = min(S_kv, -(-(q0 + Br) // Bc) * Bc) if causal else S_kv
                for tile, k0 in enumerate(range(0, kv_end, Bc)):
                    s = qt @ k[b, h, k0:k0 + Bc].T
                    if causal:
                        cols = np.arange(k0, k0 + s.shape[1])
                        s = np.where(cols[None, :] > rows[:, None], NEG_INF, s)
                    m_new = np.maximum(m, s.max(axis=-1))
                    if tile % max_every:
                        m_new = m
                    elif lazy_tau > 0:
                        m_new = np.where((m_new - m) * sl2 > np.float32(lazy_tau), m_new, m)
                    if trust_bound is not None and tile > 0:
                        # per wave: trust the running max unless the tile needs the mask or a
                        # lane's sum of p = exp2((s - m) sl2) says that some p may not fit fp16
                        if key_groups is None:
                            group = np.zeros(s.shape[1], np.int64)
                        else:
                            group = (np.arange(s.shape[1]) % key_groups[0]) // key_groups[1]
                        with np.errstate(over="ignore"):
                            p_old = np.exp2(s * sl2 - (m * sl2)[:, None], dtype=np.float32)
                            if sum_p16:
                                p_old = p_old.astype(np.float16).astype(np.float32)
                        for w0 in range(0, s.shape[0], wave_rows):
                            w = slice(w0, w0 + wave_rows)
                            if causal and k0 + s.shape[1] - 1 > q0 + w0:
                                continue
                            sums = np.stack([p_old[w][:, group == g].sum(axis=-1, dtype=np.float32)
                                             for g in range(group.max() + 1)])
                            if stats is not None:
                                stats["trusted"] = stats.get("trusted", 0) + 1
                            if np.all(sums <= np.float32(trust_bound)):
                                m_new[w] = m[w]
                            elif stats is not None:
                                stats["redone"] = stats.get("redone", 0) + 1
                    alpha = np.exp2((m - m_new) * sl2, dtype=np.float32)
                    p = np.exp2(s * sl2 - (m_new * sl2)[:, None], dtype=np.float32)
                    p16 = p.astype(np.float16).astype(np.float32)
                    l = l * alpha + (p16 if sum_p16 else p).sum(axis=-1, dtype=np.float32)
                    o = o * alpha[:, None] + p16 @ v[b, h, k0:k0 + Bc]
                    m = m_new
                out[b, h, q0:q0 + Br] = o / l[:, None]
    return out.astype(np.float16).astype(np.float32)


def attn_flops(B, H, S_q, S_kv, D, causal=False) -> float:
    f = 4.0 * B * H * S_q * S_kv * D
    return f / 2 if causal else f
