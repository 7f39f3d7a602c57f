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
    from deca_amd.kernels.rowwise_hip import regs_per_thread

    lds = 0 if cfg.threads_per_row <= arch.warp_size else 8 * cfg.threads // arch.warp_size
    wgs, _ = cu_occupancy(arch, regs_per_thread(cfg, N, op), lds, cfg.threads)
    return max(int(wgs), 1)


def rowwise_score(cfg, arch, op: str, M: int, N: int, type_size: int = 2) -> float:
    """
    Heuristic score of a memory-bound row-wise config.

    - memory parallelism: bytes of loads in flight per CU (every chunk of the
      row is requested up front in `reg` mode, `unroll` chunks in `twopass`)
      against Little's law, HBM bandwidth per CU x latency under load
      (`arch.dram_latency_s`)
    - granularity: a wave can only start reducing once all of its chunks have
      arrived and stores nothing until the row is reduced, so long per-lane chunk
      lists (few lanes per row) serialise load, math and store inside each wave;
      measured on MI355X the sweet spot is two 16-byte chunks per lane
    - wave efficiency of the grid of M / rows_per_block workgroups, and the
      drain bubble of large workgroups (all waves of a workgroup retire
      together, so 1024-lane workgroups leave wave slots idle at their tails)
    - twopass re-reads the row; the re-read hits L2 / Infinity Cache when the
      rows in flight fit
    - rows spanning several waves pay an LDS exchange and a barrier per reduction
    - idle vector lanes of the last chunk (tail) and 8-byte accesses
    - non-temporal accesses: streamed data does not displace lines in L2 /
      Infinity Cache and the writes drain earlier (measured: ~8% on MI355X)
    """
    from deca_amd.kernels.rowwise_hip import num_chunks

    wgs = rowwise_occupancy(cfg, arch, op, N)
    chunks = num_chunks(cfg, N)
    depth = chunks if cfg.mode == "reg" else cfg.unroll
    in_flight = wgs * cfg.threads * depth * cfg.vec * type_size
    need = arch.dram_bw * 1e9 / arch.sm_nums * getattr(arch, "dram_latency_s", 2e-6)
    mem = min(1.0, in_flight / need)

    # (the loss levels off: 16 and 32 chunks per lane measure the same, 0.88 of the best)
    granularity = 1.0 / (1.0 + 0.012 * min(max(0, depth - 2), 11)) * (0.985 if depth == 1 else 1.0)

    grid = M // cfg.rows_per_block
    wave_eff = _wave_efficiency(grid, arch.sm_nums * wgs)
    drain = 1.0 / (1.0 + 0.10 * max(0.0, cfg.threads / 256 - 2.0))
    rows = 1.0 / (1.0 + 0.015 * abs(math.log2(cfg.rows_per_block) - 1.0))

    passes = 1.0
    if cfg.mode == "twopass":
        footprint = arch.sm_nums * wgs * cfg.rows_per_block * N * type_size
        cache = arch.l2_bytes + getattr(arch, "mall_bytes", 0)
        hit = min(1.0, (0.8 if cfg.hint else 0.5) * cache / footprint)
        reread_bw = getattr(arch, "mall_bw", arch.l2_bw)
        passes = 1.0 + 0.5 * (hit * arch.dram_bw / reread_bw + (1.0 - hit))

    waves_per_row = max(1, cfg.threads_per_row // arch.warp_size)
    reduce = 1.0 / (1.0 + 0.005 * math.log2(waves_per_row))
    if cfg.threads_per_row < arch.warp_size:
        reduce *= 0.97

    tail = N / (chunks * cfg.threads_per_row * cfg.vec) if cfg.mode == "reg" else 1.0
    lanes = 1.0 if cfg.vec * type_size >= 16 else 0.985
    stream = 1.0 if cfg.hint else getattr(arch, "rowwise_no_hint_factor", 0.92)

    return (mem * granularity * wave_eff * drain * rows * reduce * (0.7 + 0.3 * tail) * lanes *
            stream / passes)


def rank_rowwise_configs(configs, arch, op: str, M: int, N: int, top_n: int | None = None):
    """Sort row-wise configs by `rowwise_score` (best first)."""
    ranked = sorted(configs, key=lambda c: rowwise_score(c, arch, op, M, N), reverse=True)
    return ranked[:top_n] if top_n else ranked


# ---------------------------------------------------------------------------
# FP16 MFMA GEMM
# ---------------------------------------------------------------------------
def gemm_tc_occupancy(cfg, arch) -> int:
    """Resident workgroups per CU of an FP16 MFMA GEMM config."""
    from deca_amd.kernels.gemm_hip import est_regs_per_thread, smem_bytes

    wgs, _ = cu_occupancy(arch, est_regs_per_thread(cfg), smem_bytes(cfg), cfg.threads)
    return max(int(wgs), 1)


def gemm_wave_dram_bytes_per_flop(cfg, arch, M: int, N: int, K: int, slots: int) -> float:
    """HBM bytes per FLOP of A / B (fp16) for one wave of `slots` concurrent
    workgroups.  With grouped rasterisation a wave covers `rows` workgroup rows
    x `cols` columns; every A row block and B column block of the wave is
    fetched once.  Operands that fit comfortably in the Infinity Cache are
    fetched once overall (reference: CostModel.py:182-196, with L2 -> MALL)."""
    cache = getattr(arch, "mall_bytes", arch.l2_bytes)
    if (M * K + K * N) * 2 <= 0.5 * cache:
        return (M * K + K * N) * 2 / (2.0 * M * N * K)
    GM, GN = M // cfg.BM, N // cfg.BN
    if cfg.raster == 0:  # the tiles in flight form 16 x 16 blocks
        blocks = max(1, math.ceil(min(slots, GM * GN) / 256))
        return blocks * 16 * (cfg.BM + cfg.BN) / (min(slots, GM * GN) * cfg.BM * cfg.BN)
    g = cfg.raster
    cols = min(GN, math.ceil(slots / g))
    rows = min(GM, g * math.ceil(slots / (g * GN)))
    tiles = min(slots, GM * GN)
    return (rows * cfg.BM + cols * cfg.BN) / (tiles * cfg.BM * cfg.BN)


def gemm_mma_peak(cfg, arch) -> float:
    """MFMA peak (GFLOPS) with fp32 accumulation, the only mode of the matrix cores."""
    return arch.peak_mma_sync_flops


def gemm_tc_score(cfg, arch, M: int, N: int, K: int) -> float:
    """
    Heuristic score of an FP16 MFMA GEMM config.

    Per-CU time per FLOP of the main loop, as a roofline whose non-bottleneck
    terms only partially overlap:
    - matrix cores (MFMA 32x32x16, fp32 accumulation)
    - LDS: every wave reads (WM + WN) * 16 * 2 bytes per k16 step for
      2 * WM * WN * 16 FLOPs, and the workgroup fills (BM + BN) * BK * 2 bytes
      per stage (through the LDS write port unless the loads are direct)
    - L2: every workgroup streams its A rows and B columns,
      (BM + BN) / (BM * BN) B/FLOP, from the L2 of its XCD; without the XCD remap
      neighbouring tiles land on different XCDs and share nothing there
    - HBM / Infinity Cache: the unique A / B blocks of one wave of workgroups
    - fabric: the A / B blocks that the tiles in flight on one XCD miss in its L2
    Then:
    - wave efficiency of the workgroup grid
    - issue: with one wave per SIMD nothing covers that wave's own waits (LDS
      latency before the first MFMA of a k-step, the barrier); a second wave does
    - pipelining: bytes in flight ((stages - 1) tiles per workgroup, or one tile
      for the VGPR-staged ring) vs. Little's law on the L2 stream; excess
      stages are penalised by `arch.gemm_excess_stage_penalty` (fitted on MI355X:
      a window of one 64-deep tile already saturates; deeper rings cost ~2% each)
    - one barrier per BK stage
    - epilogue: C is written once; direct stores are 8-byte row segments, the
      staged epilogue writes 16-byte coalesced chunks
    """
    wgs = gemm_tc_occupancy(cfg, arch)
    slots = arch.sm_nums * wgs
    grid = (M // cfg.BM) * (N // cfg.BN)
    wave_eff = _wave_efficiency(grid, slots)
    if getattr(cfg, "tail", False):
        # the partial last wave runs as quarter tiles: a quarter of the work each, at the
        # lower efficiency of the small tile (measured ~0.3 of a full tile's time)
        from deca_amd.kernels.gemm_hip import tail_tiles

        r = tail_tiles(cfg, M, N)
        wave_eff = (grid / slots) / ((grid - r) / slots + math.ceil(4 * r / slots) * 0.32)
    waves_per_simd = wgs * cfg.num_warps / arch.simds_per_cu
    hiding = min(1.0, 0.82 + 0.09 * min(waves_per_simd, 2.0)) if waves_per_simd >= 1 else \
        0.82 * waves_per_simd

    cus = arch.sm_nums
    wm, wn = cfg.warp_m, cfg.warp_n
    peak = gemm_mma_peak(cfg, arch)
    t_mma = cus / (peak * 1e9)
    fill_bpf = (cfg.BM + cfg.BN) / (cfg.BM * cfg.BN)
    lds_bpf = (wm + wn) / (wm * wn) + (0.0 if cfg.direct else fill_bpf)
    t_lds = lds_bpf / arch.smem_bw_per_sm
    l2_bpf = fill_bpf * (1.0 if cfg.xcd else 1.5)
    t_l2 = l2_bpf * cus / (arch.l2_bw * 1e9)
    dram_bpf = gemm_wave_dram_bytes_per_flop(cfg, arch, M, N, K, slots)
    t_dram = dram_bpf * cus / (arch.dram_bw * 1e9)
    # L2 misses: what the tiles in flight on ONE XCD need from the fabric.  A banded order
    # gives an XCD `raster` rows of tiles, the block order 8 rows by 4 columns per resident
    # workgroup; an order that is not XCD-aware leaves neighbours on different L2s.
    per_xcd = max(1, slots // getattr(arch, "num_xcd", 8))
    if not cfg.xcd:
        rows_x, cols_x = per_xcd, per_xcd
    elif cfg.raster == 0:
        rows_x, cols_x = 8, max(1, per_xcd // 8)
    else:
        rows_x = min(cfg.raster, per_xcd)
        cols_x = min(N // cfg.BN, math.ceil(per_xcd / rows_x))
    fabric_bpf = (rows_x * cfg.BM + cols_x * cfg.BN) / (per_xcd * cfg.BM * cfg.BN)
    t_fabric = fabric_bpf * cus / (getattr(arch, "mall_bw", arch.l2_bw) * 1e9)
    terms = sorted([t_mma, t_lds, t_l2, t_dram, t_fabric])
    t_flop = terms[-1] + 0.25 * sum(terms[:-1])

    # Bytes per CU that must be in flight to cover the L2 / fabric latency at the
    # sustained (power-limited, about half of peak) MFMA rate: ~0.75 us at peak rate.
    need = fill_bpf / t_mma * getattr(arch, "gemm_fill_latency_s", 0.75e-6)
    stage_bytes = wgs * (cfg.BM + cfg.BN) * cfg.BK * 2
    depth = (cfg.stages - 1) if cfg.direct else 1
    in_flight = max(depth, 0.5) * stage_bytes
    pipe = min(1.0, in_flight / need) ** 0.5
    excess = max(0, depth - math.ceil(need / stage_bytes))
    pipe *= 1.0 - getattr(arch, "gemm_excess_stage_penalty", 0.0) * excess

    # CU cycles per stage at the MFMA rate vs. ~100 cycles of barrier + refill issue
    flops_per_cycle = peak * 1e9 / cus / arch.sm_clock_hz
    stage_cycles = 2 * cfg.BM * cfg.BN * cfg.BK / flops_per_cycle
    sync_eff = 1.0 / (1.0 + 100.0 / wgs / stage_cycles)

    epi_eff = 1.0 if cfg.epi_smem else 0.5
    t_epi = (1.0 / K) / epi_eff * cus / (arch.dram_bw * 1e9)
    t_epi *= 1.0 if wgs == 1 else 0.4

    # VGPR-staged fills add global-load, LDS-write and wait instructions to the
    # MFMA issue stream (measured ~15% on MI355X)
    staged = 1.0 if cfg.direct else getattr(arch, "gemm_staged_fill_factor", 0.85)

    # 16x16x32 tiles: measured ahead of the 32x32x16 twin where the grid is a single wave of
    # workgroups or leaves a partial one (2048^3 +7 %, 4096^3 +4.5 %, 6144^3 / 10240^3 +2 %),
    # level with it on the large grids; the barrier inside the last k-step adds a little
    form = 1.0
    if getattr(cfg, "mfma", 32) == 16:
        form = 1.02 + (0.004 if getattr(cfg, "early", 0) else 0.0)
        # accumulators in accumulation registers: about 3 % over the builtin form (measured
        # at 4096^3 and 8192^3)
        if getattr(cfg, "agpr", False):
            form += 0.03
        # tile loads dealt over the MFMA groups: the more loads a wave issues per K-tile, the
        # longer the queue at the load path that the burst form makes every wave stand in
        # (measured with 8 loads per lane and K-tile: +2 % at 4096^3, +6 % at 8192^3, +7.5 %
        # at 16384^3; with 4: +1 %)
        if getattr(cfg, "spread", 0):
            loads = (cfg.BM * cfg.BK + cfg.BK * cfg.BN) // 8 // cfg.threads
            form += 0.005 * loads

    return form * wave_eff * hiding * pipe * sync_eff * staged / ((t_flop + t_epi) / t_mma)


def rank_gemm_configs(configs, arch, M: int, N: int, K: int, top_n: int | None = None,
                      per_tile: int | None = None):
    """Sort FP16 MFMA GEMM configs by `gemm_tc_score` (best first).

    `per_tile` keeps only that many tile orders (`raster`, and barrier positions `early`) of each tile set: the orders of
    one tile set score within a percent or two of each other, so that a plain top-N would
    be spent on the six orders of the one or two best tile sets."""
    ranked = sorted(configs, key=lambda c: gemm_tc_score(c, arch, M, N, K), reverse=True)
    if per_tile:
        from dataclasses import replace

        seen, kept = {}, []
        for c in ranked:
            key = replace(c, raster=1, early=0, agpr=False, spread=0)
            seen[key] = seen.get(key, 0) + 1
            if seen[key] <= per_tile:
                kept.append(c)
        ranked = kept
    return ranked[:top_n] if top_n else ranked


# ---------------------------------------------------------------------------
# FlashAttention forward
# ---------------------------------------------------------------------------
_FA_HIDDEN = 0.0  # share of a workgroup's start-up latency still exposed beside a second workgroup


def fa_occupancy(cfg, arch, D: int, grid: int):
    """Returns (resident workgroups per CU, share of the wave slots in use)."""
    from deca_amd.kernels.flash_attn_hip import est_regs_per_thread, smem_bytes

    wgs, _ = cu_occupancy(arch, est_regs_per_thread(cfg, D), smem_bytes(cfg, D), cfg.threads)
    wgs = max(int(wgs), 1)
    return wgs, wgs * cfg.num_warps / arch.max_resident_warps_per_sm


def fa_score(cfg, arch, shape, causal: bool = False) -> float:
    """
    Heuristic score of a FlashAttention config.

    - roofline of one CU per FLOP: matrix-core time vs. LDS time (every wave
      reads the whole K and V tile for its WQ query rows: 1 / WQ bytes per
      FLOP) vs. L2 time (every workgroup streams K/V once: 1 / Br bytes per
      FLOP); the non-bottleneck terms only partially overlap
    - softmax: per score element one exponential plus ~4 full rate operations
      on the vector ALU, which runs beside the matrix cores only when another
      wave on the SIMD has MFMAs to issue (or the loop interleaves them itself)
    - wave efficiency: the tail of the last wave of workgroups is wasted
    - barriers: one per KV step, hidden better by several smaller resident
      workgroups (`arch.fa_cta_sync_penalty`)
    - a 2-deep K/V ring hides the global->LDS latency; a single slot exposes it
    - causal: tiles crossing the diagonal are computed in full, so only the
      useful fraction of the computed score tiles counts
    """
    B, H, S_q, S_kv, D = shape
    grid = (S_q // cfg.Br) * B * H
    wgs, _ = fa_occupancy(cfg, arch, D, grid)
    slots = arch.sm_nums * wgs
    wave_eff = _wave_efficiency(grid, slots)

    waves_per_simd = wgs * cfg.num_warps / arch.simds_per_cu
    wq = cfg.Br // cfg.num_warps
    cus = arch.sm_nums
    t_mma = cus / (arch.peak_mma_sync_flops * 1e9)
    t_lds = (1.0 / wq) / arch.smem_bw_per_sm
    if getattr(cfg, "q_in_smem", False):
        # the wave's WQ x D Q rows are read again beside the 2 x Bc x D of K and V
        t_lds *= 1.0 + wq / (2.0 * cfg.Bc)
    t_l2 = (1.0 / cfg.Br) * cus / (arch.l2_bw * 1e9)
    # vector-ALU time per FLOP: (4 + 4) lane-cycles per score element, 4 * D FLOPs each
    valu_rate = cus * arch.simds_per_cu * 16 * arch.sm_clock_hz  # lane-ops per second
    t_valu = (8.0 / (4.0 * D)) * cus / valu_rate
    # share of the VALU work hidden under matrix work: by other waves on the SIMD,
    # or by the wave itself when its loop is software pipelined
    # (measured on MI355X: only the slot-interleaved loop adds to what a second wave
    # already hides, and even full overlap leaves ~40 % of the vector time exposed)
    overlap = min(1.0, max(0.0, waves_per_simd - 1.0) + (0.25 if int(cfg.pipe) == 2 else 0.0))
    terms = sorted([t_mma, t_lds, t_l2])
    t_flop = terms[-1] + 0.3 * (terms[0] + terms[1]) + (1.0 - 0.6 * overlap) * t_valu
    t_flop = max(t_flop, t_valu)

    pipe = 1.0 if cfg.stages >= 2 else 0.96
    # S^T one tile ahead without the slots: two S^T accumulators and a longer dependent
    # chain for nothing in return (measured 2-8 % behind the plain loop of the same tile)
    if int(cfg.pipe) == 1:
        pipe *= 0.90
    # 16x16x32 tiles, measured against the 32x32x16 twin (S = 4096): slot loop 1-2 % behind
    # on full shapes and level under the causal mask; plain loop 5-8 % ahead at D = 128 and
    # 1-2 % behind at D = 64.
    if getattr(cfg, "mfma", 32) == 16:
        if int(cfg.pipe) == 2:
            pipe *= 0.98 if not causal else 1.0
        else:
            pipe *= 1.04 if D >= 128 else 0.985
    # one copy of the two-stage plain loop: no overlap between the end of a step and the start
    # of the next (measured 1-10 % behind the unrolled form where that fits its registers; the
    # solver only emits it where the unrolled form is expected to spill)
    if getattr(cfg, "roll", False):
        pipe *= 0.99
    elif int(cfg.pipe) == 0 and cfg.stages == 2:
        from deca_amd.kernels.flash_attn_hip import register_fill

        # the unrolled form of a tile this tight is expected to spill (3-67 registers measured)
        if register_fill(cfg, D) >= 0.95:
            pipe *= 0.965
    # Measured on exhaustive runs of the S = 4096 shapes (config pairs that differ in nothing
    # else): Q fragments re-read from LDS cost 1-5 % wherever the Q-in-registers twin fits its
    # registers (they only win for tiles that would spill otherwise, which the solver's
    # register limits already drop).  Requesting tiles two steps ahead instead of one pays for
    # small K/V tiles, whose step is too short to cover a tile's latency (8 KiB: 0 ... +8 %,
    # the D = 64 winner), is level to -3 % at 16 KiB and loses beyond.
    if getattr(cfg, "q_in_smem", False):
        pipe *= 0.975
    if cfg.stages == 3:
        tile_kib = cfg.Bc * D * 2 / 1024
        pipe *= 1.015 if tile_kib <= 8 else (0.98 if tile_kib <= 16 else 0.95)
    # K/V loads dealt over the first groups of a step: +1 % in the slot loop, up to +3 % in the
    # plain loop with short (64-key, D = 64) steps, nothing or a little less elsewhere
    if getattr(cfg, "spread", 0):
        pipe *= 1.01 if int(cfg.pipe) == 2 else (1.02 if cfg.Bc * D <= 64 * 64 else 0.995)
    # no max of the tile ahead of its exponentials (plain ring loops): +3.6 % on the full
    # S = 4096 shapes at both head dims; under the causal mask nothing is gained and the
    # second pass the step keeps in reserve costs 4-7 %
    # (16x16x32 tiles then also take the row sums on the matrix pipe: another +3.9 % at D = 64,
    # +1.2 % at D = 128)
    if getattr(cfg, "trust", False):
        pipe *= 1.035 if not causal else 0.95
        if getattr(cfg, "mfma", 32) == 16 and not causal:
            pipe *= 1.035 if D < 128 else 1.01
    if not getattr(cfg, "swizzle", True):
        pipe *= 0.5  # linear LDS rows: every fragment read is a multi-way bank conflict
    sync = 1.0 / (1.0 + getattr(arch, "fa_cta_sync_penalty", 0.0) * cfg.num_warps / 4 / wgs)
    # longer KV steps amortise the per-step max / barrier; the slot loop has the row
    # statistics inside the matrix work and pays a little less of it
    step = 1.0 / (1.0 + (0.06 if int(cfg.pipe) == 2 else 0.08) * 64 / cfg.Bc)

    useful = 1.0
    if causal:
        # a wave computes every tile that reaches one of its rows in full and skips the
        # tiles beyond its last row
        nq = S_q // cfg.Br
        computed = sum(-(-(i * cfg.Br + (w + 1) * wq) // cfg.Bc) * cfg.Bc * wq
                       for i in range(nq) for w in range(cfg.num_warps))
        useful = S_q * (S_q + 1) / 2 / computed
        # The workgroups of a causal launch differ in length, and towards the end many CUs
        # hold a single one.  A workgroup that fills its SIMDs with two waves by itself keeps
        # its overlap partner until the end; a smaller one does not (measured: the causal /
        # full ratio of 4-wave configs is 0.84-0.86, of 8-wave configs 0.90).
        if cfg.num_warps < 2 * arch.simds_per_cu:
            useful *= 0.90
        # and a wave with more than one 32-query tile skips fewer masked tiles
        useful /= 1.0 + 0.15 * (wq // 32 - 1)

    # every further 32-query tile of a wave lengthens the dependent chain between barriers
    # and the prologue (twice the Q fragments): 17 % at S = 512, 2 % on long sequences
    chain = 1.0 / (1.0 + (0.02 + 0.18 * min(1.0, 512.0 / S_kv)) * (wq // 32 - 1))

    # A workgroup starts with nothing in flight (Q, then the first K/V tile) and ends with
    # the O store: a few microseconds that only another resident workgroup can cover.
    # It matters when the KV loop is short (measured at S = 512: two 4-wave workgroups per
    # CU beat one 8-wave workgroup by 20 %).  This and the other constants of this function
    # were fitted on exhaustive measurements of twelve shapes (S = 512, 1024, 4096; D = 64,
    # 128; full and causal): the measured best is then among the first 8 for all of them
    # and among the first 3 for ten.
    kv_len = S_kv * (0.5 if causal else 1.0)
    t_loop = 4.0 * cfg.Br * kv_len * D / (0.42 * arch.peak_mma_sync_flops * 1e9 / cus)
    exposed = getattr(arch, "fa_workgroup_latency_s", 4e-6) * (1.0 if wgs == 1 else _FA_HIDDEN)
    ramp = t_loop / (t_loop + exposed)

    return wave_eff * pipe * sync * step * useful * chain * ramp / (t_flop / t_mma)


def rank_fa_configs(configs, arch, shape, causal: bool = False, top_n: int | None = None):
    """Sort FlashAttention configs by `fa_score` (best first)."""
    ranked = sorted(configs, key=lambda c: fa_score(c, arch, shape, causal), reverse=True)
    return ranked[:top_n] if top_n else ranked
