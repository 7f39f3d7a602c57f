"""Host tests of the configuration solver: every emitted config is valid for
its kernel template, the enumeration is exhaustive (cross-checked against an
independent filter over the raw domain product), and the documented rules
(reg vs twopass, raster / XCD expansion) hold."""

import itertools
from dataclasses import replace

import pytest

from deca_amd import Solver
from deca_amd.arch import MI355X
from deca_amd.kernels import flash_attn_hip as fa
from deca_amd.kernels import gemm_hip as gm
from deca_amd.kernels import rowwise_hip as rw

ARCH = MI355X()


def test_intops_follow_bitvector_division():
    o = Solver._IntOps
    assert o.udiv(7, 2) == 3 and o.urem(7, 2) == 1
    assert o.udiv(7, 0) == 2**32 - 1 and o.urem(7, 0) == 7
    assert o.implies(False, False) and not o.implies(True, False)
    assert o.ite(True, 1, 2) == 1 and o.all_of(True, True) and o.any_of(False, True)


@pytest.mark.parametrize("op,M,N", [("softmax", 16384, 4096), ("rmsnorm", 16384, 4096),
                                    ("rmsnorm", 8192, 8192), ("softmax", 4096, 1024),
                                    ("softmax", 1024, 32000), ("softmax", 8192, 128256)])
def test_rowwise_configs_are_valid_and_exhaustive(op, M, N):
    configs = Solver.solve_rowwise(ARCH, op, M, N)
    assert configs and len(set(configs)) == len(configs)
    for cfg in configs:
        rw.check_config(cfg, op, M, N, "float16")
        assert M // cfg.rows_per_block >= ARCH.sm_nums
        assert cfg.threads_per_row * cfg.vec <= N
    # independent enumeration: raw product filtered by the kernel's own rules
    want = set()
    for tpr, rpb, vec, mode, unroll, hint in itertools.product(
            (16, 32, 64, 128, 256, 512, 1024), (1, 2, 4, 8, 16), (4, 8), ("reg", "twopass"),
            (1, 2, 4), (False, True)):
        cfg = rw.RowConfig(tpr, rpb, vec, mode, unroll, hint)
        try:
            rw.check_config(cfg, op, M, N, "float16")
        except AssertionError:
            continue
        if M // rpb < ARCH.sm_nums or tpr * vec > N:
            continue
        if mode == "reg" and (unroll != 1 or rw.num_chunks(cfg, N) > 32):
            continue
        if rw.regs_per_thread(cfg, N, op) > ARCH.max_arch_vgprs:
            continue
        want.add(cfg)
    has_reg = any(c.mode == "reg" for c in want)
    if N < 16384 and has_reg:
        want = {c for c in want if c.mode == "reg"}
    assert set(configs) == want


def test_rowwise_mode_rules():
    assert all(c.mode == "reg" for c in Solver.solve_rowwise(ARCH, "softmax", 16384, 4096))
    modes = {c.mode for c in Solver.solve_rowwise(ARCH, "softmax", 1024, 32000)}
    assert modes == {"reg", "twopass"}  # N >= 16384: both offered
    # a row too long for the register file: only twopass survives
    long_row = Solver.solve_rowwise(ARCH, "softmax", 1024, 1 << 19)
    assert long_row and {c.mode for c in long_row} == {"twopass"}
    # lowering the threshold admits twopass for short rows too
    both = Solver.solve_rowwise(ARCH, "softmax", 16384, 4096, twopass_min_n=1024)
    assert {c.mode for c in both} == {"reg", "twopass"}
    assert len(Solver.solve_rowwise(ARCH, "softmax", 16384, 4096, count=5)) == 5
    assert Solver.solve_rowwise(ARCH, "softmax", 64, 4096) == []  # fewer rows than CUs


@pytest.mark.parametrize("n", [2048, 4096, 8192])
def test_gemm_configs_are_valid(n):
    configs = Solver.solve_gemm_tc(ARCH, n, n, n)
    assert configs and len(set(configs)) == len(configs)
    for cfg in configs:
        gm.check_config(cfg, n, n, n)
        assert (n // cfg.BM) * (n // cfg.BN) >= ARCH.sm_nums
        full = (n // cfg.BM) * (n // cfg.BN) - (gm.tail_tiles(cfg, n, n) if cfg.tail else 0)
        if cfg.raster == 0:  # 8 x 4 sub-blocks of tiles per XCD, whole rounds of 8 of them
            assert cfg.xcd and (n // cfg.BM) % 8 == 0 and (n // cfg.BN) % 4 == 0 and full % 256 == 0
        else:
            assert (n // cfg.BM) % cfg.raster == 0
        assert cfg.xcd == (full % 8 == 0)
        assert cfg.stages >= 2 if cfg.direct else cfg.stages <= 2
    if n >= 4096:
        assert gm.GemmConfig(256, 256, 64, 128, 64, 2, 4, False, True, True) in configs
    # independent enumeration of the tile sets
    tiles = set()
    for bm, bn, bk, wm, wn, st, epi, direct, mfma in itertools.product(
            (64, 128, 256), (64, 128, 256), (32, 64), (32, 64, 128), (32, 64, 128), (1, 2, 3, 4, 5),
            (False, True), (False, True), (32, 16)):
        if bm % wm or bn % wn:
            continue
        xcd = ((n // bm) * (n // bn)) % 8 == 0
        cfg = gm.GemmConfig(bm, bn, bk, wm, wn, st, 1, epi, xcd, direct, mfma=mfma)
        try:
            gm.check_config(cfg, n, n, n)
        except AssertionError:
            continue
        if (n // bm) * (n // bn) < ARCH.sm_nums:
            continue
        regs = (gm.est_regs_per_thread(cfg) + 7) // 8 * 8
        if regs * -(-cfg.num_warps // 4) > 512 or gm.est_regs_per_thread(cfg) > gm.SPILL_FREE_EST_REGS:
            continue
        tiles.add((bm, bn, bk, wm, wn, st, epi, direct, mfma))
    got = {(c.BM, c.BN, c.BK, c.warp_m, c.warp_n, c.stages, c.epi_smem, c.direct, c.mfma)
           for c in configs}
    assert got == tiles
    # the 16x16x32 body offers its barrier before or in the middle of a tile's last k-step
    assert {c.early for c in configs if c.mfma == 16 and c.warp_m == 128} == {0, 4}
    assert all(c.early == 0 for c in configs if c.mfma == 32)
    # every rasterisation that divides the grid is offered for every tile set
    for c in configs:
        if c.tail:
            continue
        gm_, gn_ = n // c.BM, n // c.BN
        want = {r for r in (1, 2, 4, 8, 16) if gm_ % r == 0}
        if gm_ % 8 == 0 and gn_ % 4 == 0 and (gm_ * gn_) % 256 == 0:
            want.add(0)
        have = {d.raster for d in configs if not d.tail and
                (d.BM, d.BN, d.BK, d.warp_m, d.warp_n, d.stages, d.epi_smem, d.direct, d.mfma, d.early)
                == (c.BM, c.BN, c.BK, c.warp_m, c.warp_n, c.stages, c.epi_smem, c.direct, c.mfma, c.early)}
        assert have == want
        break


def test_gemm_rejects_shapes_no_tile_divides():
    assert Solver.solve_gemm_tc(ARCH, 4096 + 8, 4096, 4096) == []


@pytest.mark.parametrize("D,S", [(128, 4096), (64, 4096), (128, 512)])
def test_flash_attn_configs_are_valid(D, S):
    B, H = (4, 16) if S == 4096 else (32, 16)
    configs = Solver.solve_flash_attn(ARCH, B, H, S, S, D)
    assert configs and len(set(configs)) == len(configs)
    for cfg in configs:
        fa.check_config(cfg, S, S, D)
        assert (S // cfg.Br) * B * H >= ARCH.sm_nums
    want = set()
    for br, bc, nw, st, pipe, mfma, qs in itertools.product(
            (32, 64, 128, 256), (32, 64, 128), (1, 2, 4, 8), (1, 2, 3), (0, 1, 2), (32, 16), (0, 1)):
        cfg = fa.FAConfig(br, bc, nw, st, pipe=pipe, mfma=mfma, q_in_smem=bool(qs))
        try:
            fa.check_config(cfg, S, S, D)
        except AssertionError:
            continue
        if (S // br) * B * H < ARCH.sm_nums or st > S // bc or (pipe and S // bc < 2):
            continue
        regs = (fa.est_regs_per_thread(cfg, D) + 7) // 8 * 8
        if regs * -(-nw // 4) > 512 or not fa.expect_spill_free(cfg, D):
            continue
        forms = [cfg]
        # the one-copy form of the plain ring loop, where the unrolled one is tight
        if pipe == 0 and st >= 2 and fa.register_fill(cfg, D) >= 0.95:
            forms.append(replace(cfg, roll=True))
        # the load window of the two-stage plain and slot loops
        if st == 2 and pipe in (0, 2):
            forms.append(replace(cfg, spread=8 if pipe == 2 else 4))
        # every plain ring loop also without the tile's max ahead of its exponentials
        if pipe == 0 and st >= 2:
            forms += [replace(f, trust=True) for f in forms]
        want.update(forms)
    assert set(configs) == want
    assert all(int(c.pipe) == 0 and c.stages >= 2 for c in configs if c.trust)
    # the reference's knobs are all in the search (Solver.py:330-336), except linear LDS rows
    assert {c.stages for c in configs} == {1, 2, 3}
    assert {c.q_in_smem for c in configs} == {False, True} and all(c.swizzle for c in configs)
    assert all(fa.smem_bytes(c, D) <= ARCH.max_dyn_smem_per_block for c in configs)
    # a tighter register budget removes the widest per-wave tiles
    tight = Solver.solve_flash_attn(ARCH, B, H, S, S, D, max_est_regs=256)
    assert set(tight) < set(configs) or set(tight) == set(configs)
    assert all(fa.est_regs_per_thread(c, D) <= 256 for c in tight)


def test_flash_attn_register_limits_follow_the_compiler():
    """The per-loop-shape limits on the register estimate: just below them hipcc
    allocates without spilling, the first estimate above them spills."""
    from deca_amd.kernels.build import kernel_resources

    def resources(cfg, D):
        return kernel_resources(fa.make_flash_attn_fwd(4, 16, 4096, 4096, D, cfg, None, False))

    keep = fa.FAConfig(256, 64, 4, 1)   # D = 128: estimate 352 <= 365, one LDS stage
    drop = fa.FAConfig(256, 64, 4, 2)   # same tile, two stages: limit 330
    assert fa.expect_spill_free(keep, 128) and not fa.expect_spill_free(drop, 128)
    configs = Solver.solve_flash_attn(ARCH, 4, 16, 4096, 4096, 128)
    assert keep in configs and drop not in configs
    assert resources(keep, 128)["vgpr_spills"] == 0
    assert resources(drop, 128)["vgpr_spills"] > 0
    slots = fa.FAConfig(256, 64, 4, 2, pipe=2)  # estimate 384 <= 480
    assert slots in configs
    got = resources(slots, 128)
    assert got["vgpr_spills"] == 0 and got["scratch_bytes"] == 0


def test_z3_backend_agrees_with_enumeration():
    pytest.importorskip("z3")
    a = Solver.solve_rowwise(ARCH, "softmax", 16384, 4096, backend="z3")
    b = Solver.solve_rowwise(ARCH, "softmax", 16384, 4096, backend="enumerate")
    assert a == b
    a = Solver.solve_flash_attn(ARCH, 4, 16, 4096, 4096, 128, backend="z3")
    b = Solver.solve_flash_attn(ARCH, 4, 16, 4096, 4096, 128, backend="enumerate")
    assert a == b


def test_z3_backend_is_reported_missing():
    if Solver._z3 is not None:
        pytest.skip("z3 is installed")
    with pytest.raises(RuntimeError, match="z3"):
        Solver.solve_rowwise(ARCH, "softmax", 16384, 4096, backend="z3")


def test_slot_interleaved_loop_needs_paired_key_blocks():
    """`pipe == 2` issues the S^T chains in pairs of 32-key blocks and must fit the
    exponentials ahead of the O^T instructions that consume them."""
    assert all(fa.slot_schedule_ok(bc, d) for bc in (64, 128) for d in (64, 128))
    assert not any(fa.slot_schedule_ok(bc, d) for bc in (32, 96) for d in (64, 128))
    fa.check_config(fa.FAConfig(128, 64, 4, 2, pipe=2), 512, 512, 128)
    with pytest.raises(AssertionError):
        fa.check_config(fa.FAConfig(128, 32, 4, 2, pipe=2), 512, 512, 128)
    with pytest.raises(AssertionError):
        fa.check_config(fa.FAConfig(128, 64, 4, 1, pipe=2), 512, 512, 128)
    assert str(fa.FAConfig(128, 64, 4, 2, pipe=2)).endswith(",pipe=2")
    assert str(fa.FAConfig(128, 64, 4, 2, pipe=True)).endswith(",pipe=1")
    picked = Solver.solve_flash_attn(ARCH, 4, 16, 4096, 4096, 128)
    assert any(c.pipe == 2 for c in picked) and all(c.Bc % 64 == 0 for c in picked if c.pipe == 2)


def test_kernels_are_compiled_for_the_occupancy_the_estimates_allow():
    """A workgroup of 4 waves or fewer must not be given the whole register file when the
    LDS has room for a second one (DECA_MIN_WAVES)."""
    from deca_amd.kernels import gemm_hip as gm

    # D = 64: two 4-wave workgroups fit the LDS and 256 registers each
    small = fa.FAConfig(256, 64, 4, 2)
    assert fa.est_regs_per_thread(small, 64) <= 256 and fa.target_waves_per_simd(small, 64) == 2
    # D = 128, 4 waves with two query tiles each: more than 256 registers -> one wave per SIMD
    assert fa.target_waves_per_simd(fa.FAConfig(256, 64, 4, 2), 128) == 1
    # 8 waves are two per SIMD by themselves; a 128 KiB ring leaves no room for more
    assert fa.target_waves_per_simd(fa.FAConfig(256, 128, 8, 2), 128) == 2
    spec = fa.make_flash_attn_fwd(1, 8, 512, 512, 64, small, None, False)
    assert dict(spec.defines)["DECA_MIN_WAVES"] == 2
    big = gm.GemmConfig(256, 256, 64, 128, 64, 2, 8, True, True, True)
    assert gm.target_waves_per_simd(big) == 2
    assert gm.target_waves_per_simd(gm.GemmConfig(128, 256, 64, 64, 128, 2, 8, True, True, True)) == 1
    assert dict(gm.make_gemm_tc(4096, 4096, 4096, big).defines)["DECA_MIN_WAVES"] == 2


def test_flash_attn_rolled_loop_is_offered_where_registers_are_tight():
    cfgs = Solver.solve_flash_attn(ARCH, 4, 16, 4096, 4096, 128)
    rolled = {c for c in cfgs if c.roll}
    assert fa.FAConfig(256, 128, 8, 2, mfma=16, roll=True) in rolled
    assert all(",roll=1" in str(c) and replace(c, roll=False) in cfgs for c in rolled)
    assert fa.FAConfig(256, 64, 8, 2, roll=True) not in rolled  # 204 of 256 registers: room enough
    assert dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, next(iter(rolled))).defines)["DECA_ROLL"] == 1
    with pytest.raises(AssertionError):
        fa.check_config(fa.FAConfig(256, 64, 8, 2, pipe=2, roll=True), 4096, 4096, 128)


def test_flash_attn_knobs_of_the_reference():
    """`q_in_smem`, `swizzle` and `stages` 1..3 (flash_attn_tir.py:35-38) all reach the
    kernel: LDS footprint, register estimate and the macros of the specialisation."""
    base = fa.FAConfig(256, 64, 8, 2)
    staged = replace(base, q_in_smem=True)
    assert fa.smem_bytes(base, 128) == 2 * 2 * 64 * 128 * 2
    assert fa.smem_bytes(staged, 128) == fa.smem_bytes(base, 128) + 256 * 128 * 2
    # all D/16 fragments of a query tile against two in flight (flash_attn_tir.py:65)
    assert fa.est_regs_per_thread(base, 128) - fa.est_regs_per_thread(staged, 128) == (128 // 16 - 2) * 4
    defs = dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, staged).defines)
    assert defs["DECA_QSMEM"] == 1 and "DECA_SWIZZLE" not in defs
    defs = dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, replace(base, swizzle=False)).defines)
    assert defs["DECA_SWIZZLE"] == 0 and "DECA_QSMEM" not in defs
    deep = fa.FAConfig(128, 64, 4, 3)
    spec = fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, deep)
    assert dict(spec.defines)["DECA_STAGES"] == 3 and dict(spec.meta)["no_scratch"] is True
    assert dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, base).meta)["no_scratch"] is False
    assert str(staged).find("q_smem=1") > 0 and str(replace(base, swizzle=False)).find("swz=0") > 0
    # the winner tile of D = 128 (a 128 KiB ring) has no room for a 64 KiB Q tile
    with pytest.raises(AssertionError):
        fa.check_config(fa.FAConfig(256, 128, 8, 2, q_in_smem=True), 4096, 4096, 128)
    # the spread load window: two-stage plain and slot loops only
    assert fa.default_spread(base) == 4 and fa.default_spread(replace(base, pipe=2)) == 8
    assert fa.default_spread(deep) == 0 and fa.default_spread(replace(base, roll=True)) == 0
    fa.check_config(replace(deep, spread=4), 4096, 4096, 128)  # accepted, just not offered
    sp = replace(base, pipe=2, spread=8)
    assert dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, sp).defines)["DECA_SPREAD"] == 8
    assert str(sp).endswith(",pipe=2,spread=8")
    for bad in (replace(base, pipe=1, spread=4), replace(base, stages=1, spread=4)):
        with pytest.raises(AssertionError):
            fa.check_config(bad, 4096, 4096, 128)
    # no max ahead of a tile's exponentials: plain ring loops only (the slot loop consumes
    # P while the check is still out, the one-stage loop has no ring step to repeat in)
    tr = replace(base, mfma=16, roll=True, trust=True)
    assert dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, tr).defines)["DECA_TRUST"] == 1
    assert "DECA_TRUST" not in dict(fa.make_flash_attn_fwd(4, 16, 4096, 4096, 128, base).defines)
    assert str(tr).endswith(",mfma=16,roll=1,trust=1")
    fa.check_config(replace(deep, trust=True), 4096, 4096, 128)
    for bad in (replace(base, pipe=2, trust=True), replace(base, pipe=1, trust=True),
                replace(base, stages=1, trust=True)):
        with pytest.raises(AssertionError):
            fa.check_config(bad, 4096, 4096, 128)
    # three stages belong to the plain loop; four do not exist
    for bad in (fa.FAConfig(128, 64, 4, 3, pipe=2), fa.FAConfig(128, 64, 4, 3, pipe=1), fa.FAConfig(128, 64, 4, 4)):
        with pytest.raises(AssertionError):
            fa.check_config(bad, 4096, 4096, 128)


def test_flash_attn_head_dims():
    """Every multiple of 64 is supported, as in the reference (flash_attn_tir.py:70-72);
    anything else yields no config instead of a bad one."""
    for D in (192, 256, 320):
        wide = Solver.solve_flash_attn(ARCH, 4, 16, 2048, 2048, D)
        assert wide
        for cfg in wide:
            fa.check_config(cfg, 2048, 2048, D)
    assert Solver.solve_flash_attn(ARCH, 4, 16, 2048, 2048, 96) == []
    with pytest.raises(AssertionError):
        fa.check_config(fa.FAConfig(128, 64, 4, 2), 2048, 2048, 96)


def test_gemm_accumulation_register_twins():
    """16x16x32 configs whose registers split evenly between the two halves of the file come
    with an `agpr=1` twin; nothing else does."""
    cfgs = Solver.solve_gemm_tc(ARCH, 4096, 4096, 4096)
    twins = [c for c in cfgs if c.agpr]
    assert twins and all(c.mfma == 16 and ",agpr=1" in str(c) and replace(c, agpr=False) in cfgs
                         and gm.agpr_split_fits(c) for c in twins)
    big = gm.GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, mfma=16, early=4, agpr=True)
    assert big in twins
    spec = gm.make_gemm_tc(4096, 4096, 4096, big)
    assert dict(spec.defines)["DECA_ACC_AGPR"] == 1
    # 128 accumulators cleared once and read once
    assert dict(spec.meta)["accumulator_moves"] == 2 * 128 == gm.accumulator_moves(big)
    assert gm.accumulator_moves(replace(big, tail=True)) == 2 * (128 + 32)
    with pytest.raises(AssertionError):
        gm.check_config(replace(big, mfma=32, early=0), 4096, 4096, 4096)


def test_gemm_tail_split_is_offered_where_a_partial_wave_remains():
    """6144^3 with 256 x 256 tiles: 576 tiles = 2 waves of 256 + 64; the 64 may run as 256
    quarter tiles.  A grid that fills its waves exactly gets no such variant."""
    cfgs = Solver.solve_gemm_tc(ARCH, 6144, 6144, 6144)
    split = [c for c in cfgs if c.tail]
    assert split and all(",tail=1" in str(c) for c in split)
    big = gm.GemmConfig(256, 256, 64, 128, 64, 2, 8, True, True, True, tail=True)
    assert big in split and gm.tail_tiles(big, 6144, 6144) == 64
    spec = gm.make_gemm_tc(6144, 6144, 6144, big)
    assert spec.grid == (512 + 4 * 64, 1, 1)
    assert dict(spec.defines)["DECA_TAIL"] == 64 and dict(spec.defines)["DECA_TAIL_STAGES"] == 4
    for c in split:
        gm.check_config(c, 6144, 6144, 6144)
        assert 0 < gm.tail_tiles(c, 6144, 6144)
    assert gm.GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, tail=True) in split
    # 8192^3 with the same tile: 1024 tiles = 4 full waves
    with pytest.raises(AssertionError):
        gm.check_config(big, 8192, 8192, 8192)
    assert not any(c.tail and (c.BM, c.BN) == (256, 256) for c in Solver.solve_gemm_tc(ARCH, 8192, 8192, 8192))
    # the cost model prefers the split at 6144 and scores a config without tail as before
    from deca_amd.cost_model import CostModel as cm

    plain = gm.GemmConfig(256, 256, 64, 128, 64, 2, 8, True, True, True)
    assert cm.gemm_tc_score(big, ARCH, 6144, 6144, 6144) > cm.gemm_tc_score(plain, ARCH, 6144, 6144, 6144)


def test_gemm_spread_twins():
    """Every 16x16x32 config whose K-tile has six or more MFMA groups comes with a twin whose
    tile loads are dealt over the groups (`spread`); the 32x32x16 body has none."""
    from deca_amd import tuned

    cfgs = set(Solver.solve_gemm_tc(ARCH, 4096, 4096, 4096))
    twins = [c for c in cfgs if c.spread]
    assert twins and all(c.mfma == 16 and c.direct and replace(c, spread=0) in cfgs for c in twins)
    assert all(c.spread == gm.default_spread(c) for c in twins)
    def valid(c):
        try:
            gm.check_config(c, 4096, 4096, 4096)
            return True
        except AssertionError:
            return False

    for c in cfgs:
        if c.mfma == 16 and not c.spread and gm.default_spread(c):
            twin = replace(c, spread=gm.default_spread(c))
            assert (twin in cfgs) == valid(twin), c
    big = gm.GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, mfma=16, early=4, agpr=True, spread=6)
    assert big in cfgs and gm.mfma_groups_per_ktile(big) == 16 and gm.default_spread(big) == 6
    small = gm.GemmConfig(128, 128, 64, 64, 32, 4, 4, True, True, True, mfma=16, early=2)
    assert gm.mfma_groups_per_ktile(small) == 8 and gm.default_spread(small) == 3
    assert gm.default_spread(gm.GemmConfig(64, 64, 32, 32, 64, 2, 2, False, False, True, mfma=16)) == 0
    spec = gm.make_gemm_tc(4096, 4096, 4096, big)
    defs, meta = dict(spec.defines), dict(spec.meta)
    assert defs["DECA_DMA_SPREAD"] == 6 and defs["DECA_DMA_FIRST"] == gm.SPREAD_FIRST == 1
    assert meta["no_scratch"] is True  # the prologue waits for part of its loads
    plain = dict(gm.make_gemm_tc(4096, 4096, 4096, replace(big, spread=0)).defines)
    assert "DECA_DMA_SPREAD" not in plain
    assert str(big).endswith(",agpr=1,spread=6") and tuned.parse_config("GEMM", str(big)) == big
    with pytest.raises(AssertionError):  # the 32x32x16 body issues its loads in one burst
        gm.check_config(gm.GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, spread=6), 4096, 4096, 4096)
    with pytest.raises(AssertionError):  # more groups than a K-tile has
        gm.check_config(replace(big, spread=16), 4096, 4096, 4096)


def test_gemm_spread_prologue_fits_the_load_counter():
    """With `spread` the prologue leaves the head of the second tile in flight beside the
    (stages - 2) youngest tiles; the host mirrors the kernel's count, and the solver drops the
    deep one-wave rings where the 6-bit counter would overflow."""
    assert gm.spread_head_loads(8, 8, 2, 4, 6) == 4      # 256 x 256 x 64, 8 waves: half a tile
    assert gm.spread_head_loads(8, 8, 2, 4, 0) == 0
    assert gm.spread_head_loads(16, 4, 2, 0, 3) == 16    # window shorter than the groups behind the barrier
    deep = gm.GemmConfig(64, 64, 64, 64, 64, 5, 1, True, True, True, mfma=16, agpr=True, spread=3)
    with pytest.raises(AssertionError):
        gm.check_config(deep, 2048, 2048, 2048)          # 3 x 16 + 16 loads in flight
    gm.check_config(replace(deep, spread=0), 2048, 2048, 2048)
    cfgs = Solver.solve_gemm_tc(ARCH, 2048, 2048, 2048)
    assert deep not in cfgs and replace(deep, spread=0) in cfgs
    for c in cfgs:
        if c.spread:
            loads = (c.BM * c.BK + c.BK * c.BN) // 8 // c.threads
            head = gm.spread_head_loads(loads, c.warp_m // 16, c.BK // 32, c.early, c.spread)
            assert (c.stages - 2) * loads + head <= 63
