"""
Analytical ranking of kernel configurations (larger score = expected faster).

Same entry points as the reference's src/cost_model/CostModel.py
(`rank_rowwise_configs` :280, `rank_gemm_configs` :274, `rank_fa_configs` :96
and the `*_score` / `*_occupancy` helpers); the terms are re-derived for a
CDNA4 compute unit.  Only the ordering of the top-N matters: measurement picks
the winner.
"""

from __future__ import annotations

import math

from deca_amd.driver.driver import cu_occupancy


class CostModel:
    """Kept for interface compatibility (reference: CostModel.py:7-12 is an empty stub)."""

    def cost(self, kernel, arch, compute_pattern):
        raise NotImplementedError("use the rank_* functions of this module")


def _wave_efficiency(grid: int, slots: int) -> float:
    """Useful share of the launch's workgroup waves: the tail of the last wave idles."""
    waves = math.ceil(grid / slots)
    return grid / (waves * slots)


# ---------------------------------------------------------------------------
# row-wise
# ---------------------------------------------------------------------------
def rowwise_occupancy(cfg, arch, op: str, N: int) -> int:
    """Resident workgroups per CU of a row-wise (Softmax / RMSNorm) config."""
    from deca_amd.kernels.rowwise_hip import est_regs_per_thread

    lds = 0 if cfg.threads_per_row <= arch.warp_size else 8 * cfg.threads // arch.warp_size
    wgs, _ = cu_occupancy(arch, est_regs_per_thread(cfg, N, op), lds, cfg.threads)
    return max(int(wgs), 1)


def rowwise_score(cfg, arch, op: str, M: int, N: int, type_size: int = 2) -> float:
    """
    Heuristic score of a memory-bound row-wise config.

    - memory parallelism: bytes of loads in flight per CU (every chunk of the
      row is requested up front in `reg` mode, `unroll` chunks in `twopass`)
      against Little's law, HBM bandwidth per CU x latency under load
      (`arch.dram_latency_s`)
    - phases: a workgroup loads, reduces, then stores; with few resident
      workgroups per CU the reduce/store phase is not hidden by other loads
    - wave efficiency of the grid of M / rows_per_block workgroups
    - twopass re-reads the row; the re-read hits L2 / Infinity Cache when the
      rows in flight fit
    - rows spanning several waves pay an LDS exchange and a barrier per
      reduction; rows narrower than a wave idle no lanes but shorten bursts
    - idle vector lanes of the last chunk (tail) and 8-byte accesses
    - non-temporal accesses keep the streamed data from displacing reusable lines
    """
    from deca_amd.kernels.rowwise_hip import num_chunks

    wgs = rowwise_occupancy(cfg, arch, op, N)
    chunks = num_chunks(cfg, N)
    per_lane = (chunks if cfg.mode == "reg" else cfg.unroll) * cfg.vec * type_size
    in_flight = wgs * cfg.threads * per_lane
    need = arch.dram_bw * 1e9 / arch.sm_nums * getattr(arch, "dram_latency_s", 2e-6)
    mem = min(1.0, in_flight / need)

    phase = 1.0 - (0.35 if cfg.mode == "reg" else 0.1) / wgs

    grid = M // cfg.rows_per_block
    wave_eff = _wave_efficiency(grid, arch.sm_nums * wgs)

    passes = 1.0
    if cfg.mode == "twopass":
        footprint = arch.sm_nums * wgs * cfg.rows_per_block * N * type_size
        cache = arch.l2_bytes + getattr(arch, "mall_bytes", 0)
        hit = min(1.0, (0.8 if cfg.hint else 0.5) * cache / footprint)
        reread_bw = getattr(arch, "mall_bw", arch.l2_bw)
        passes = 1.0 + 0.5 * (hit * arch.dram_bw / reread_bw + (1.0 - hit))

    waves_per_row = max(1, cfg.threads_per_row // arch.warp_size)
    reduce = 1.0 / (1.0 + 0.02 * math.log2(waves_per_row) + (0.03 if waves_per_row > 1 else 0.0))
    if cfg.threads_per_row < arch.warp_size:
        reduce *= 0.97

    tail = N / (chunks * cfg.threads_per_row * cfg.vec) if cfg.mode == "reg" else 1.0
    lanes = 1.0 if cfg.vec * type_size >= 16 else 0.97
    stream = 1.0 if cfg.hint else getattr(arch, "rowwise_no_hint_factor", 0.96)

    return mem * phase * wave_eff * reduce * (0.7 + 0.3 * tail) * lanes * stream / passes


def rank_rowwise_configs(configs, arch, op: str, M: int, N: int, top_n: int | None = None):
    """Sort row-wise configs by `rowwise_score` (best first)."""
    ranked = sorted(configs, key=lambda c: rowwise_score(c, arch, op, M, N), reverse=True)
    return ranked[:top_n] if top_n else ranked
