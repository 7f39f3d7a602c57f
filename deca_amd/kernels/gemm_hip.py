"""
FP16 MFMA GEMM (C = A @ B, fp32 accumulation): config type, resource estimates,
validity rules and the specialisation of the HIP template `csrc/gemm.hip`.

Counterpart of the reference's src/kernels/gemm_tir.py.  Layout: A[M, K],
B[K, N], C[M, N], all row-major float16.

What changes on CDNA4 (reference mechanism -> here):
- mma.sync.m16n8k16 (gemm_tir.py:280-290) -> v_mfma_f32_32x32x16_f16 or (`mfma=16`)
  v_mfma_f32_16x16x32_f16; a wave is 64 lanes and owns a `warp_m x warp_n` tile made of
  32x32 (16x16) MFMA tiles;
- ldmatrix / ldmatrix.trans (:262-278) -> ds_read_b128 for A and the transposing
  ds_read_b64_tr_b16 for the row-major B tile;
- cp.async ring (:190-199) -> asynchronous 16-byte global -> LDS loads that bypass the
  VGPRs (`direct`, ring of 2 to 5 K-tiles, explicit vmcnt waits), or 16-byte global loads
  staged through VGPRs one K-tile ahead of the MFMAs into a 1- or 2-deep LDS ring;
- 128-byte-line XOR swizzle (:14-18) -> chunk swizzles sized for the 64-bank LDS;
- grouped rasterisation (:159-163) -> the same grouping applied after dealing
  contiguous tile ranges to the 8 XCDs (each has a private L2);
- fp16 accumulation (`acc_f16`, `acc_splits`, :52-58) has no MFMA counterpart
  (the matrix cores always accumulate in fp32) and is not offered.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass

from deca_amd.kernels.build import (
    DEFAULT_ARCH, FAST_MATH_OPTIONS, KernelSpec, build_kernel, cached_build, make_spec,
)

WAVE = 64
MFMA_M = 32  # v_mfma_f32_32x32x16_f16
MFMA_K = 16
MAX_VGPRS = 512  # unified VGPRs (arch + accumulation) per lane at one wave per SIMD
MAX_LDS = 160 * 1024
# Padding (halves) of the epilogue staging rows.
EPI_PAD = 8
TEMPLATE = "gemm.hip"


@dataclass(frozen=True)
class GemmConfig:
    BM: int = 256  # workgroup tile rows
    BN: int = 256  # workgroup tile columns
    BK: int = 64  # K depth of one pipeline stage
    warp_m: int = 128  # wave tile rows
    warp_n: int = 128  # wave tile columns
    stages: int = 2  # LDS ring depth: 2..4 with direct loads, 1..2 with VGPR staging
    # workgroup rows per rasterisation group (1: plain row-major order); 0: every XCD works
    # on an 8 x 4 sub-block of tiles, and the 8 sub-blocks in flight are neighbours
    raster: int = 8
    epi_smem: bool = False  # stage C through LDS for 16-byte stores
    xcd: bool = True  # deal contiguous tile ranges to the 8 XCDs
    direct: bool = True  # global -> LDS loads that bypass the VGPRs (else VGPR-staged)
    # the tiles of the partial last wave of workgroups are split into four quarter tiles
    # (BM/2 x BN/2, wave tiles halved), so that they fill the whole GPU for a quarter of
    # a tile's time instead of a quarter of the GPU for a whole one
    tail: bool = False
    # MFMA tile: 32 -> v_mfma_f32_32x32x16, 16 -> v_mfma_f32_16x16x32 (less energy per
    # FLOP on this board; needs BK = 64 and the direct-to-LDS ring)
    mfma: int = 32
    # 16x16x32 body: row-block groups of a K-tile's last k-step that issue before the
    # barrier which publishes the next tile (a later barrier gives the loads more time,
    # and leaves fewer MFMAs to cover the first fragment reads of the next tile)
    early: int = 0
    # 16x16x32 body: accumulators tied to accumulation registers (AGPRs), the MFMAs written
    # as inline assembly (about 3 % faster than the builtin form; the build step checks the
    # generated code, see `accumulator_moves`)
    agpr: bool = False
    # 16x16x32 body: the global->LDS loads of a tile are dealt over this many MFMA groups
    # instead of issued in one burst at the top of a K-tile (0).  All waves of a workgroup
    # leave the K-tile barrier together and queue up at the CU's one load path (a 64-lane x
    # 16-byte load per 16 clocks); a wave in that queue issues no MFMA.  The window of a
    # tile opens one group behind the barrier that frees its ring slot and runs into the
    # next K-tile (measured: +2 % at 4096^3, +6 % at 8192^3, +7.5 % at 16384^3 with 6).
    spread: int = 0

    @property
    def num_warps(self) -> int:
        return (self.BM // self.warp_m) * (self.BN // self.warp_n)

    @property
    def threads(self) -> int:
        return self.num_warps * WAVE

    def as_dict(self):
        return asdict(self)

    def __str__(self):
        return (
            f"{self.BM}x{self.BN}x{self.BK},warp={self.warp_m}x{self.warp_n},"
            f"stages={self.stages},raster={self.raster},epi_smem={int(self.epi_smem)}"
            + ("" if self.xcd else ",xcd=0")
            + ("" if self.direct else ",direct=0")
            + (",tail=1" if self.tail else "")
            + (f",mfma={self.mfma}" if self.mfma != 32 else "")
            + (f",early={self.early}" if self.early else "")
            + (",agpr=1" if self.agpr else "")
            + (f",spread={self.spread}" if self.spread else "")
        )


# Groups behind a K-tile's barrier that pass before the first load of the spread window.
SPREAD_FIRST = 1


def mfma_groups_per_ktile(cfg: GemmConfig) -> int:
    """MFMA groups (one row block against every column block) of a K-tile in the 16x16x32 body."""
    return (cfg.BK // 32) * (cfg.warp_m // 16)


def spread_head_loads(loads: int, mt: int, ks: int, early: int, spread: int) -> int:
    """Loads of the second tile that the prologue issues with `spread` (what the groups
    behind a barrier would have issued of it), as the kernel computes it: the window has
    `ks * mt` groups, the first `mt - early` of them lie behind the barrier, and the loads
    are dealt over `spread` groups starting `SPREAD_FIRST` groups in."""
    if not spread:
        return 0
    groups = ks * mt
    early = min(early, mt - 1)
    post = mt - early
    n = min(spread, groups)
    first = SPREAD_FIRST if SPREAD_FIRST + n <= groups else groups - n
    if post <= first:
        return 0
    return loads if post - first >= n else (post - first) * loads // n


def default_spread(cfg: GemmConfig) -> int:
    """The window the solver offers for a tile: 6 groups where a K-tile has 12 or more
    (measured best of 2..12 for 256 x 256 x 64 tiles), 3 where it has 6 or more, else none --
    and none where the register estimate fills the budget of the waves that share a SIMD to
    the last eight registers: such a build spills a few registers (64 x 128 wave tiles of the
    builtin 16x16x32 body: 8-44 bytes), and with the load window's partial wait in the
    prologue the loader refuses a build that spills."""
    if (est_regs_per_thread(cfg) + 8) * -(-cfg.num_warps // 4) > MAX_VGPRS:
        return 0
    groups = mfma_groups_per_ktile(cfg)
    return 6 if groups >= 12 else (3 if groups >= 6 else 0)


def pipeline_smem_bytes(cfg: GemmConfig) -> int:
    return cfg.stages * (cfg.BM * cfg.BK + cfg.BK * cfg.BN) * 2


def epilogue_smem_bytes(cfg: GemmConfig) -> int:
    return cfg.BM * (cfg.BN + EPI_PAD) * 2 if cfg.epi_smem else 0


def smem_bytes(cfg: GemmConfig) -> int:
    """The epilogue reuses the pipeline buffers once the main loop is done."""
    return max(pipeline_smem_bytes(cfg), epilogue_smem_bytes(cfg))


# Largest register estimate hipcc was seen to allocate without spilling: the estimate
# tracks the compiler's allocation within a few registers up to here; the tile sets
# above it (128 x 128 wave tiles staged through registers) spill in the main loop.
SPILL_FREE_EST_REGS = 456


def est_regs_per_thread(cfg: GemmConfig) -> int:
    """Unified VGPR estimate per lane: fp32 accumulators (warp_m * warp_n / 64),
    one set of A / B fragments (4 VGPRs per 32-row tile), the global->LDS
    staging registers and addressing."""
    acc = cfg.warp_m * cfg.warp_n // WAVE
    chunks = (cfg.BM * cfg.BK + cfg.BK * cfg.BN) // 8 // cfg.threads
    # direct loads keep one offset register per chunk, staged loads four data registers
    staging = chunks if cfg.direct else chunks * 4
    if cfg.mfma == 16:
        # one set of A fragments (refilled in place), two of B, 4 VGPRs per 16-row tile
        return acc + 4 * (cfg.warp_m // 16 + 2 * (cfg.warp_n // 16)) + staging + 40
    frags = 4 * (cfg.warp_m // MFMA_M + cfg.warp_n // MFMA_M)  # one of the two sets
    return acc + 2 * frags + staging + 40


NUM_CUS = 256  # gfx950 (MI355X)


def resident_workgroups(cfg: GemmConfig) -> int:
    """Workgroups of this config one CU holds at a time (registers, LDS, 32 wave slots)."""
    regs8 = (est_regs_per_thread(cfg) + 7) // 8 * 8
    waves = cfg.threads // WAVE
    by_regs = (512 // regs8) // -(-waves // 4)
    return max(1, min(by_regs, MAX_LDS // smem_bytes(cfg), 32 // waves))


def tail_tiles(cfg: GemmConfig, M: int, N: int) -> int:
    """Tiles of the partial last wave: what is left when the grid is dealt to the
    workgroup slots of the whole GPU."""
    return ((M // cfg.BM) * (N // cfg.BN)) % (NUM_CUS * resident_workgroups(cfg))


def tail_stages(cfg: GemmConfig) -> int:
    """Ring depth of the quarter tiles: twice the slots fit the same LDS."""
    return min(4 if cfg.direct else 2, 2 * cfg.stages)


def agpr_split_fits(cfg: GemmConfig) -> bool:
    """Whether the 16x16x32 body is expected to build with its accumulators in accumulation
    registers: the compiler then gives each half of the register file half of a wave's
    budget, so the accumulators and everything else must each fit their half."""
    acc = (cfg.warp_m // 16) * (cfg.warp_n // 16) * 4
    half = (512 // target_waves_per_simd(cfg)) // 2
    return cfg.mfma == 16 and acc <= half and est_regs_per_thread(cfg) - acc <= half - 8


def accumulator_moves(cfg: GemmConfig) -> int:
    """`v_accvgpr_*` instructions a kernel with `agpr` accumulators may contain: one write per
    accumulator register to clear it and one read in the epilogue, for the full tile and,
    with `tail`, for the quarter tile.  The compiler does not know that the asm statements
    are matrix instructions and would not wait for one before it moves an accumulator; a
    build with any further move is refused (`build.check_generated_code`)."""
    regs = (cfg.warp_m // 16) * (cfg.warp_n // 16) * 4
    if cfg.tail:
        regs += (cfg.warp_m // 32) * (cfg.warp_n // 32) * 4
    return 2 * regs


def target_waves_per_simd(cfg: GemmConfig) -> int:
    """Waves per SIMD the kernel is compiled for: what the estimated registers and the LDS
    footprint let co-reside.  The compiler only knows the block size, and gives a workgroup
    of 4 waves or fewer the whole 512-register file even when the LDS has room for a second
    workgroup on the same SIMDs."""
    regs8 = (est_regs_per_thread(cfg) + 7) // 8 * 8
    by_regs = 512 // regs8
    by_lds = (MAX_LDS // smem_bytes(cfg)) * (cfg.threads // WAVE) // 4
    return max(1, min(by_regs, by_lds, 8))


def check_config(cfg: GemmConfig, M: int, N: int, K: int, max_smem: int = MAX_LDS) -> None:
    assert cfg.stages in ((2, 3, 4, 5) if cfg.direct else (1, 2))
    assert K // cfg.BK >= cfg.stages
    assert smem_bytes(cfg) <= max_smem
    assert cfg.BK in (32, 64)
    assert cfg.mfma in (32, 16)
    if cfg.mfma == 16:
        # k-steps of 32; with one k-step per K-tile the main loop takes two tiles at a time
        assert cfg.direct
        assert cfg.BK == 64 or (K // cfg.BK) % 2 == 0
        assert 0 <= cfg.early < cfg.warp_m // 16
        # 64 accumulator tiles of 16 x 16 per wave: hipcc fills all 256 accumulation and
        # all 256 vector registers and still spills 30-170 inside the loop (8x slower)
        assert (cfg.warp_m // 16) * (cfg.warp_n // 16) <= 32
        assert 0 <= cfg.spread <= mfma_groups_per_ktile(cfg) - SPREAD_FIRST
    else:
        assert cfg.early == 0 and not cfg.agpr and cfg.spread == 0
    assert cfg.warp_m % MFMA_M == 0 and cfg.warp_n % MFMA_M == 0
    assert cfg.BM % cfg.warp_m == 0 and cfg.BN % cfg.warp_n == 0
    assert cfg.BN >= 64
    assert M % cfg.BM == 0 and N % cfg.BN == 0 and K % cfg.BK == 0
    assert WAVE <= cfg.threads <= 1024
    # Every lane issues the same number of 16-byte loads for each operand.
    assert (cfg.BM * cfg.BK // 8) % cfg.threads == 0
    assert (cfg.BK * cfg.BN // 8) % cfg.threads == 0
    if cfg.direct:
        # loads left in flight by the (stages - 2) youngest tiles -- and, with `spread`, the
        # head of the next one in the prologue -- fit the 6-bit counter
        loads = (cfg.BM * cfg.BK + cfg.BK * cfg.BN) // 8 // cfg.threads
        head = spread_head_loads(loads, cfg.warp_m // 16, cfg.BK // 32, cfg.early, cfg.spread)
        assert (cfg.stages - 2) * loads + head <= 63
    if cfg.tail:
        r = tail_tiles(cfg, M, N)
        tiles = (M // cfg.BM) * (N // cfg.BN)
        assert 0 < r < tiles
        assert not cfg.xcd or (tiles - r) % 8 == 0
        assert (cfg.warp_m // 2) % MFMA_M == 0 and (cfg.warp_n // 2) % MFMA_M == 0 and cfg.BN // 2 >= 64
        assert (cfg.BM // 2 * cfg.BK // 8) % cfg.threads == 0
        assert (cfg.BK * (cfg.BN // 2) // 8) % cfg.threads == 0
        assert not cfg.epi_smem or (cfg.BM // 2 * (cfg.BN // 2) // 8) % cfg.threads == 0
        qs = tail_stages(cfg)
        assert K // cfg.BK >= qs
        if cfg.direct:
            q_loads = (cfg.BM // 2 * cfg.BK + cfg.BK * (cfg.BN // 2)) // 8 // cfg.threads
            q_head = spread_head_loads(q_loads, max(1, cfg.warp_m // 32), cfg.BK // 32, cfg.early, cfg.spread)
            assert (qs - 2) * q_loads + q_head <= 63
    if cfg.raster == 0:
        full = (M // cfg.BM) * (N // cfg.BN) - (tail_tiles(cfg, M, N) if cfg.tail else 0)
        assert cfg.xcd and (M // cfg.BM) % 8 == 0 and (N // cfg.BN) % 4 == 0 and full % 256 == 0
    else:
        assert (M // cfg.BM) % cfg.raster == 0
    if cfg.xcd:  # the remap permutes the full tiles
        full = (M // cfg.BM) * (N // cfg.BN) - (tail_tiles(cfg, M, N) if cfg.tail else 0)
        assert full % 8 == 0
    if cfg.epi_smem:
        assert (cfg.BM * cfg.BN // 8) % cfg.threads == 0
    assert est_regs_per_thread(cfg) <= MAX_VGPRS


DTYPES = ("float16", "bfloat16")


def make_gemm_tc(M: int, N: int, K: int, cfg: GemmConfig, dtype: str = "float16") -> KernelSpec:
    """Specialised kernel: 1-D grid of (M/BM)*(N/BN) workgroups of `threads`
    lanes (reference: gemm_tir.py:156), static LDS.  `dtype` is the type of A, B
    and C (the reference is fp16 only; bf16 uses the bf16 MFMA of the same shape)."""
    check_config(cfg, M, N, K)
    assert dtype in DTYPES
    defines = {
        "DECA_M": M, "DECA_N": N, "DECA_K": K,
        "DECA_BM": cfg.BM, "DECA_BN": cfg.BN, "DECA_BK": cfg.BK,
        "DECA_WM": cfg.warp_m, "DECA_WN": cfg.warp_n,
        "DECA_STAGES": cfg.stages, "DECA_RASTER": cfg.raster,
        "DECA_EPI_LDS": int(cfg.epi_smem), "DECA_XCD": int(cfg.xcd),
        "DECA_DIRECT": int(cfg.direct), "DECA_BF16": int(dtype == "bfloat16"),
        "DECA_MIN_WAVES": target_waves_per_simd(cfg),
    }
    if cfg.mfma == 16:
        defines["DECA_MFMA16"] = 1
        defines["DECA_EARLY_GROUPS"] = cfg.early
    if cfg.agpr:
        defines["DECA_ACC_AGPR"] = 1
    if cfg.spread:
        defines["DECA_DMA_SPREAD"] = cfg.spread
        defines["DECA_DMA_FIRST"] = SPREAD_FIRST
    workgroups = (M // cfg.BM) * (N // cfg.BN)
    if cfg.tail:
        r = tail_tiles(cfg, M, N)
        defines["DECA_TAIL"] = r
        defines["DECA_TAIL_STAGES"] = tail_stages(cfg)
        workgroups += 3 * r
    return make_spec(
        TEMPLATE, defines, grid=(workgroups, 1, 1), block=(cfg.threads, 1, 1),
        nargs=3, options=FAST_MATH_OPTIONS,
        # the direct-load ring waits with vmcnt(n > 0) once it is deeper than two tiles
        # (the quarter tiles of `tail` always are; with `spread` the prologue does, for the
        # head of the second tile): the loader refuses a build that spills
        meta={"cfg": str(cfg), "dtype": dtype,
              "no_scratch": bool(cfg.direct and (cfg.stages > 2 or cfg.tail or cfg.spread)),
              **({"accumulator_moves": accumulator_moves(cfg)} if cfg.agpr else {})},
    )


GEMM_HIPCC_OPTIONS = FAST_MATH_OPTIONS


def build_gemm_tc(spec: KernelSpec, target: str | None = None, dump_dir: str | None = None):
    """Compiles (or takes from the in-tree cache) and loads the kernel;
    `dump_dir` keeps the generated ISA for inspection."""
    import os

    from deca_amd.driver.driver import load_kernel

    arch = target or DEFAULT_ARCH
    if dump_dir:
        path = build_kernel(spec, arch, os.path.join(dump_dir, f"gemm_{spec.key()}.hsaco"), dump_dir)
    else:
        path = cached_build(spec, arch)
    return load_kernel(spec, path)


def build_gemm_tc_to_file(shape, cfg: GemmConfig, arch: str, path: str,
                          dtype: str = "float16") -> str:
    """Builds in a worker process (no GPU context needed) and writes a code object."""
    M, N, K = shape
    return build_kernel(make_gemm_tc(M, N, K, cfg, dtype), arch, path)
