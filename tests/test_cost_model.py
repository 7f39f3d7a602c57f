"""Host tests of the analytical ranking: occupancy arithmetic checked by hand,
closed-form pieces, and the monotonic behaviour each term is there for."""

import math

import pytest

from deca_amd.arch import MI355X
from deca_amd.cost_model import CostModel as cm
from deca_amd.driver.driver import cu_occupancy
from deca_amd.kernels.flash_attn_hip import FAConfig
from deca_amd.kernels.gemm_hip import GemmConfig
from deca_amd.kernels.rowwise_hip import RowConfig

ARCH = MI355X()


def test_cu_occupancy_by_hand():
    # 256 lanes = 4 waves = one per SIMD; 128 VGPRs -> 4 waves per SIMD -> 4 workgroups
    assert cu_occupancy(ARCH, 128, 0, 256) == (4, 4)
    # 64 VGPRs -> 8 waves per SIMD (the cap), 32 waves per CU / 4 per workgroup
    assert cu_occupancy(ARCH, 64, 0, 256) == (8, 8)
    # more than 256 VGPRs: one wave per SIMD
    assert cu_occupancy(ARCH, 300, 0, 256) == (1, 1)
    # LDS bound: 64 KiB per workgroup -> 2 workgroups in 160 KiB
    assert cu_occupancy(ARCH, 64, 64 * 1024, 256)[0] == 2
    # a single-wave workgroup: 4 SIMDs x 5 waves of 100 (-> 104) VGPRs... 512 // 104 = 4
    assert cu_occupancy(ARCH, 100, 0, 64) == (16, 4)
    # 512 lanes = 8 waves = 2 per SIMD; 250 (-> 256) VGPRs -> 2 waves per SIMD -> 1 workgroup
    assert cu_occupancy(ARCH, 250, 0, 512) == (1, 2)
    assert cu_occupancy(ARCH, 600, 0, 64) == (0, 0)


def test_wave_efficiency():
    assert cm._wave_efficiency(512, 256) == 1.0
    assert cm._wave_efficiency(257, 256) == pytest.approx(257 / 512)


def test_rowwise_score_terms():
    M, N = 16384, 4096
    base = RowConfig(128, 1, 8)
    s0 = cm.rowwise_score(base, ARCH, "softmax", M, N)
    assert 0 < s0 <= 1
    # non-temporal hints, 16-byte accesses and reg mode each help
    assert cm.rowwise_score(RowConfig(128, 1, 8, hint=True), ARCH, "softmax", M, N) > s0
    assert cm.rowwise_score(RowConfig(128, 1, 4), ARCH, "softmax", M, N) < s0
    assert cm.rowwise_score(RowConfig(128, 1, 8, "twopass", 2), ARCH, "softmax", M, N) < s0
    # a ragged tail idles lanes
    assert cm.rowwise_score(base, ARCH, "softmax", M, 4104) < s0
    ranked = cm.rank_rowwise_configs([RowConfig(1024, 1, 4), base], ARCH, "softmax", M, N, top_n=1)
    assert ranked == [base]
    assert cm.rowwise_occupancy(RowConfig(64, 1, 8), ARCH, "softmax", N) >= 1


def test_gemm_dram_bytes_per_flop_closed_form():
    cfg = GemmConfig(256, 256, 64, 128, 64, 2, 4)
    # operands that fit half the Infinity Cache are fetched once overall
    n = 4096
    assert cm.gemm_wave_dram_bytes_per_flop(cfg, ARCH, n, n, n, 256) == pytest.approx(
        (2 * n * n * 2) / (2.0 * n**3))
    # large problem: one wave of 256 tiles in groups of 4 rows covers 4 rows x 64 columns
    n = 16384
    got = cm.gemm_wave_dram_bytes_per_flop(cfg, ARCH, n, n, n, 256)
    assert got == pytest.approx((4 * 256 + 64 * 256) / (256 * 256 * 256))


def test_gemm_score_terms():
    n = 8192
    good = GemmConfig(256, 256, 64, 128, 64, 2, 4)
    s = cm.gemm_tc_score(good, ARCH, n, n, n)
    assert 0 < s <= 1
    # small tiles need more LDS and L2 bytes per FLOP
    assert cm.gemm_tc_score(GemmConfig(64, 64, 64, 32, 32, 2, 4), ARCH, n, n, n) < s
    # a staged ring pays the LDS write traffic that direct loads avoid
    assert cm.gemm_tc_score(GemmConfig(256, 256, 64, 128, 64, 2, 4, direct=False), ARCH, n, n, n) < s
    # without the XCD remap the L2 term grows
    assert cm.gemm_tc_score(GemmConfig(256, 256, 64, 128, 64, 2, 4, xcd=False), ARCH, n, n, n) <= s
    assert cm.gemm_tc_occupancy(good, ARCH) == 1
    top = cm.rank_gemm_configs([GemmConfig(64, 64, 64, 32, 32, 2, 4), good], ARCH, n, n, n, top_n=1)
    assert top == [good]
    assert cm.gemm_mma_peak(good, ARCH) == ARCH.peak_mma_sync_flops


def test_fa_score_terms():
    shape = (4, 16, 4096, 4096, 128)
    a = FAConfig(256, 128, 8, 2)
    s = cm.fa_score(a, ARCH, shape)
    assert s > 0
    assert cm.fa_score(FAConfig(256, 128, 8, 1), ARCH, shape) < s       # single slot exposes latency
    assert cm.fa_score(a, ARCH, shape, causal=True) < s                  # diagonal tiles are wasted work
    # causal useful fraction: a wave computes the tiles that reach its 32 rows in full
    one = FAConfig(256, 128, 8, 1)
    nq, computed = 4096 // 256, 0
    for i in range(nq):
        for w in range(8):
            computed += math.ceil((i * 256 + (w + 1) * 32) / 128) * 128 * 32
    ratio = cm.fa_score(one, ARCH, shape, True) / cm.fa_score(one, ARCH, shape, False)
    # ... times the start-up latency of a workgroup, which weighs more on the halved KV loop
    rate = 0.42 * ARCH.peak_mma_sync_flops * 1e9 / ARCH.sm_nums
    t_full, lat = 4.0 * 256 * 4096 * 128 / rate, 4e-6
    ramp = (t_full / 2 / (t_full / 2 + lat)) / (t_full / (t_full + lat))
    assert ratio == pytest.approx(4096 * 4097 / 2 / computed * ramp)
    # a short KV loop favours two resident workgroups over one that owns the CU
    short = (32, 16, 512, 512, 128)
    assert (cm.fa_score(FAConfig(128, 64, 4, 2), ARCH, short) / cm.fa_score(a, ARCH, short)
            > cm.fa_score(FAConfig(128, 64, 4, 2), ARCH, shape) / cm.fa_score(a, ARCH, shape))
    # the loop shapes: S^T one tile ahead without the slots trails the plain loop, the slot
    # loop leads it; a causal launch costs the small workgroups their overlap partner
    b = FAConfig(256, 64, 8, 2)
    assert (cm.fa_score(FAConfig(256, 64, 8, 2, pipe=1), ARCH, shape) < cm.fa_score(b, ARCH, shape)
            < cm.fa_score(FAConfig(256, 64, 8, 2, pipe=2), ARCH, shape))
    small = FAConfig(128, 64, 4, 2)
    assert (cm.fa_score(small, ARCH, shape, True) / cm.fa_score(small, ARCH, shape)
            < cm.fa_score(b, ARCH, shape, True) / cm.fa_score(b, ARCH, shape))
    # 16x16x32 tiles: just behind the 32x32x16 twin in the slot loop, ahead of it in the plain
    # loop at D = 128, behind it at D = 64 (as measured)
    assert cm.fa_score(FAConfig(256, 64, 8, 2, pipe=2, mfma=16), ARCH, shape) == pytest.approx(
        0.98 * cm.fa_score(FAConfig(256, 64, 8, 2, pipe=2), ARCH, shape))
    assert cm.fa_score(FAConfig(256, 64, 8, 2, mfma=16), ARCH, shape) > cm.fa_score(FAConfig(256, 64, 8, 2), ARCH, shape)
    d64 = (4, 16, 4096, 4096, 64)
    assert cm.fa_score(FAConfig(256, 64, 4, 2, mfma=16), ARCH, d64) < cm.fa_score(FAConfig(256, 64, 4, 2), ARCH, d64)
    wgs, share = cm.fa_occupancy(a, ARCH, 128, 1024)
    assert wgs == 1 and share == pytest.approx(8 / 32)
    assert cm.rank_fa_configs([FAConfig(32, 32, 1, 1), a], ARCH, shape, top_n=1) == [a]


def test_gemm_ranking_can_limit_the_tile_orders_per_tile_set():
    from dataclasses import replace

    from deca_amd import Solver

    n = 8192
    cfgs = Solver.solve_gemm_tc(ARCH, n, n, n)
    plain = cm.rank_gemm_configs(cfgs, ARCH, n, n, n, top_n=12)
    spread = cm.rank_gemm_configs(cfgs, ARCH, n, n, n, top_n=12, per_tile=3)
    tiles = lambda cs: {replace(c, raster=1, early=0) for c in cs}  # noqa: E731
    assert len(tiles(spread)) >= 4 > len(tiles(plain)) - 1
    assert spread[0] == plain[0]
    for t in tiles(spread):
        assert sum(replace(c, raster=1, early=0) == t for c in spread) <= 3
    # the order of what is kept is still the score order
    scores = [cm.gemm_tc_score(c, ARCH, n, n, n) for c in spread]
    assert scores == sorted(scores, reverse=True)


def test_rank_report_reads_the_drivers_output():
    """The rank-quality table is made from the text the tuning drivers print."""
    from deca_amd.cost_model import rank_report as rr

    def rec(what, cfg, ms, thr, unit):
        return f"{what} \n\t{cfg} \n\tcost time: {ms:.4f} ms, throughput: {thr:.2f} {unit}, max err: 1.00e-04\n"

    text = "Detected GPU: X\nFind 244 FlashAttention configs, measuring 4\n"
    fa = "FlashAttention(B=4, H=16, S_q=4096, S_kv=4096, D=128, float16)"
    for cfg, thr in (("Br=256,Bc=128", 1000.0), ("Br=256,Bc=64", 1100.0), ("Br=128,Bc=64", 900.0),
                     ("Br=64,Bc=64", 500.0)):
        text += rec(fa, cfg, 0.5, thr, "TFLOPS")
    text += "Br=32,Bc=32 is not a valid config: spills\n✅✅✅ 2026-01-01 [X]\n DeCA ...\n"
    text += "Find 80 Softmax configs, measuring 2\n"
    sm = "Softmax(M=16384, N=4096, float16)"
    text += rec(sm, "tpr=256,rpb=2", 0.042, 6300.0, "GB/s") + rec(sm, "tpr=128,rpb=1", 0.05, 5300.0, "GB/s")
    runs = rr.parse_runs(text)
    assert [r["what"] for r in runs] == [fa, sm]
    assert runs[0]["solutions"] == 244 and len(runs[0]["measured"]) == 4 and runs[1]["unit"] == "GB/s"
    q = rr.quality(runs[0])
    assert q["best_rank"] == 2 and q["best_cfg"] == "Br=256,Bc=64"
    assert abs(q["first"] - 1000 / 1100) < 1e-9 and q["top3"] == 1.0
    assert rr.spearman([4.0, 3.0, 2.0, 1.0]) == 1.0 and rr.spearman([1.0, 2.0, 3.0, 4.0]) == -1.0
    assert rr.quality(runs[1])["best_rank"] == 1
    lines = rr.table(runs).splitlines()
    assert len(lines) == 4 and "| 244 | 4 | 2 |" in lines[2]


def test_rank_report_pairs_configurations_that_differ_in_one_field():
    """`pair_effects`: ratios over twins that differ in one field, also for a field that is
    only printed when it is set (an empty old value)."""
    from deca_amd.cost_model import rank_report as rr

    run = {"what": "x", "solutions": 6, "unit": "TFLOPS", "measured": [
        ("Br=256,stages=2", 1000.0), ("Br=256,stages=3", 900.0), ("Br=256,stages=2,trust=1", 1040.0),
        ("Br=128,stages=2", 500.0), ("Br=128,stages=2,trust=1", 490.0), ("Br=64,stages=3,trust=1", 100.0)]}
    e = rr.pair_effects(run, "stages=2", "stages=3")
    assert e["pairs"] == 1 and abs(e["median"] - 0.9) < 1e-12
    e = rr.pair_effects(run, "", "trust=1")
    assert e["pairs"] == 2 and abs(e["min"] - 0.98) < 1e-12 and abs(e["max"] - 1.04) < 1e-12
    assert e["near_pairs"] == 1 and e["top"] == ("Br=256,stages=2,trust=1", 1040.0, 1000.0)
    assert " -> trust=1 | 2 |" in rr.pairs_table([run], [":trust=1"])
