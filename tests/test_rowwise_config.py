"""Host logic of the row-wise kernels: config rules, geometry, compile-only."""

import os

import pytest

from deca_amd.kernels import rowwise_hip as rw
from deca_amd.kernels.build import kernel_resources
from deca_amd.kernels.rowwise_hip import RowConfig


def test_str_is_the_log_key():
    assert str(RowConfig()) == "tpr=128,rpb=1,vec=8,mode=reg"
    assert str(RowConfig(256, 2, 4, "twopass", 4, True)) == "tpr=256,rpb=2,vec=4,mode=twopass,unroll=4,hint=1"
    assert RowConfig(64, 4).threads == 256
    assert hash(RowConfig()) == hash(RowConfig(128, 1, 8, "reg", 1, False))


def test_num_chunks():
    assert rw.num_chunks(RowConfig(128, 1, 8), 4096) == 4
    assert rw.num_chunks(RowConfig(128, 1, 8), 4104) == 5
    assert rw.num_chunks(RowConfig(1024, 1, 8), 128256) == 16


@pytest.mark.parametrize("cfg,ok", [
    (RowConfig(128, 1, 8), True),
    (RowConfig(32, 1, 8), False),       # 32 threads: not a whole wave
    (RowConfig(32, 2, 8), True),
    (RowConfig(1024, 2, 8), False),     # 2048 threads
    (RowConfig(128, 3, 8), False),      # M % rpb
    (RowConfig(96, 2, 8), False),       # tpr not a power of two
    (RowConfig(128, 1, 8, "twopass", 8), False),  # unroll > full chunks (4)
    (RowConfig(128, 1, 2, hint=True), False),     # hints need >= 8-byte accesses
])
def test_check_config(cfg, ok):
    if ok:
        rw.check_config(cfg, "softmax", 16384, 4096, "float16")
    else:
        with pytest.raises(AssertionError):
            rw.check_config(cfg, "softmax", 16384, 4096, "float16")


def test_geometry_and_macros():
    spec = rw.make_rowwise("rmsnorm", 16384, 4096, "bfloat16", RowConfig(256, 2, 8), 1e-5)
    assert spec.grid == (8192, 1, 1) and spec.block == (512, 1, 1) and spec.nargs == 3
    d = dict(spec.defines)
    assert d["DECA_OP"] == 1 and d["DECA_BF16"] == 1 and d["DECA_N"] == 4096 and d["DECA_EPS"] == "1e-05"
    assert rw.make_rowwise("softmax", 64, 1024, "float16", RowConfig(64, 1, 8)).nargs == 2


def test_compile_only_and_register_estimate(tmp_path):
    """hipcc cross-compiles for gfx950 without a GPU; the estimator tracks the
    recorded VGPR count closely enough for occupancy ranking."""
    for op, dtype, cfg in [("softmax", "float16", RowConfig(128, 1, 8)),
                           ("rmsnorm", "bfloat16", RowConfig(256, 1, 8)),
                           ("softmax", "bfloat16", RowConfig(64, 2, 8, "twopass", 2, True))]:
        spec = rw.make_rowwise(op, 16384, 4096, dtype, cfg)
        res = kernel_resources(spec)
        assert res["vgpr_spills"] == 0 and res["scratch_bytes"] == 0
        est = rw.est_regs_per_thread(cfg, 4096, op)
        assert abs(est - res["vgprs"]) <= 0.5 * res["vgprs"] + 8
    path = rw.build_rowwise_to_file("softmax", (64, 1024), "float16", RowConfig(64, 1, 8), 1e-6,
                                    "gfx950", str(tmp_path / "k.hsaco"))
    assert os.path.getsize(path) > 1000


def test_lean_reg_mode_is_chosen_when_the_plain_one_does_not_fit(tmp_path):
    """A 128256-element row over 1024 lanes is 128 elements per lane: the plain reg mode
    (fp32 values kept between the passes) does not fit 16 waves into the register files,
    the lean one (packed row only) does, and compiles without spills."""
    cfg = RowConfig(1024, 1, 8, "reg", 1, True)
    for op, dtype in (("softmax", "float16"), ("rmsnorm", "bfloat16")):
        assert rw.use_lean(cfg, 128256, op) and not rw.use_lean(cfg, 32000, op)
        rw.check_config(cfg, op, 4096, 128256, dtype)
        spec = rw.make_rowwise(op, 4096, 128256, dtype, cfg)
        assert dict(spec.defines)["DECA_LEAN"] == 1
        res = kernel_resources(spec)
        assert res["vgpr_spills"] == 0 and res["scratch_bytes"] == 0
        assert res["vgprs"] <= rw.lean_regs_per_thread(cfg, 128256) <= 128
    assert "DECA_LEAN" not in dict(rw.make_rowwise("softmax", 4096, 32000, "float16", cfg).defines)
    # 64 chunks per lane are beyond the unrolled row loop
    with pytest.raises(AssertionError):
        rw.check_config(RowConfig(256, 1, 8, "reg"), "softmax", 4096, 128256, "float16")
    # the solver offers the register-cached form for vocabulary-size rows
    from deca_amd import Solver
    from deca_amd.arch.MI355X import MI355X

    cfgs = Solver.solve_rowwise(MI355X(), "softmax", 4096, 128256)
    assert cfg in cfgs and any(c.mode == "twopass" for c in cfgs)
