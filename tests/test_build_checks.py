"""The build step checks what a kernel spec promises about its generated code."""

import pytest

from deca_amd.kernels.build import build_kernel, check_generated_code
from deca_amd.kernels.gemm_hip import GemmConfig, make_gemm_tc


def _spec(early):
    cfg = GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, mfma=16, early=early, agpr=True)
    return make_gemm_tc(4096, 4096, 4096, cfg)


def test_accumulator_move_count_is_checked_on_the_text():
    spec = _spec(4)
    ok = "\n".join(["\tv_accvgpr_write_b32 a0, 0"] * 128 + ["\tv_accvgpr_read_b32 v1, a0"] * 128
                   + ["    .vgpr_spill_count: 0", "    .private_segment_fixed_size: 0"])
    check_generated_code(spec, ok)
    with pytest.raises(RuntimeError, match="accumulation-register moves"):
        check_generated_code(spec, ok + "\n\tv_accvgpr_mov_b32 a4, a8")
    with pytest.raises(RuntimeError):
        check_generated_code(spec, ok.replace(".vgpr_spill_count: 0", ".vgpr_spill_count: 3"))
    # a spec without the promise is not looked at
    check_generated_code(make_gemm_tc(4096, 4096, 4096, GemmConfig(256, 256, 64, 128, 64, 2, 0, True)), "")


def test_late_operand_writes_are_found_on_the_text():
    from deca_amd.kernels.build import late_operand_writes

    mfma = "\tv_mfma_f32_16x16x32_f16 a[0:3], v[4:7], v[8:11], a[0:3]\n"
    write = "\tv_mov_b32_e32 v5, v9\n"
    assert late_operand_writes(write + mfma)                       # no wait state between
    assert late_operand_writes(write + "\ts_nop 0\n" + mfma)       # one
    assert not late_operand_writes(write + "\ts_nop 1\n" + mfma)   # two
    assert not late_operand_writes(write + "\tds_read_b128 v[20:23], v1\n\ts_waitcnt lgkmcnt(0)\n" + mfma)
    assert not late_operand_writes("\tv_mov_b32_e32 v50, v9\n" + mfma)  # another register
    # an MFMA the compiler wrote itself (vector-register result) gets its wait states from it
    assert not late_operand_writes(write + "\tv_mfma_f32_16x16x32_f16 v[0:3], v[4:7], v[8:11], v[0:3]\n")
    spec = _spec(4)
    text = "\n".join(["\tv_accvgpr_write_b32 a0, 0"] * 128 + ["\tv_accvgpr_read_b32 v1, a0"] * 128) + "\n"
    with pytest.raises(RuntimeError, match="two wait states"):
        check_generated_code(spec, text + write + mfma)


def test_build_refuses_a_kernel_whose_accumulators_the_compiler_moves(tmp_path):
    """256 x 256 x 64 with the barrier after two row blocks: hipcc runs out of vector registers
    in its half of the file and shuffles accumulators inside the loop (measured: wrong
    results).  The same tile with the barrier after four row blocks builds."""
    good = build_kernel(_spec(4), None, str(tmp_path / "good.hsaco"))
    assert (tmp_path / "good.hsaco").exists() and good.endswith("good.hsaco")
    with pytest.raises(RuntimeError, match="accumulation-register moves"):
        build_kernel(_spec(2), None, str(tmp_path / "bad.hsaco"))
    assert not (tmp_path / "bad.hsaco").exists()


def test_a_shared_dump_dir_cannot_lend_its_assembly_to_another_build(tmp_path):
    """The checked assembly is this build's own: a dump directory that already holds other
    kernels' files (one of them sorting after the GEMM's) changes neither the verdict nor
    what is kept."""
    from deca_amd.kernels.rowwise_hip import RowConfig, make_rowwise

    dump = tmp_path / "dump"
    dump.mkdir()
    stale = dump / "rowwise-hip-amdgcn-amd-amdhsa-gfx950.s"
    stale.write_text("\tv_accvgpr_mov_b32 a4, a8\n")           # would fail the check if it were read
    (dump / "gemm-hip-amdgcn-amd-amdhsa-gfx950.s").write_text("stale\n")
    spec = _spec(4)
    build_kernel(spec, None, str(tmp_path / "g.hsaco"), str(dump))
    kept = dump / f"gemm_{spec.key()}.s"
    assert kept.exists() and "v_mfma_f32_16x16x32" in kept.read_text()
    assert stale.read_text() == "\tv_accvgpr_mov_b32 a4, a8\n"
    # a refused build leaves nothing of its own behind
    bad = _spec(2)
    with pytest.raises(RuntimeError, match="accumulation-register moves"):
        build_kernel(bad, None, str(tmp_path / "b.hsaco"), str(dump))
    assert not (dump / f"gemm_{bad.key()}.s").exists()
    # unchecked builds keep their assembly the same way
    row = make_rowwise("softmax", 256, 4096, "float16", RowConfig(128, 1, 8), 1e-6)
    build_kernel(row, None, str(tmp_path / "r.hsaco"), str(dump))
    assert (dump / f"rowwise_{row.key()}.s").exists()


def test_checked_kernels_are_tied_to_the_validated_compiler(monkeypatch):
    from deca_amd.kernels import build

    spec = _spec(4)
    assert build.hipcc_version().startswith(build.VALIDATED_HIPCC)
    build.require_validated_hipcc(spec)
    monkeypatch.setattr(build, "_hipcc_version", "HIP version: 9.9.0-deadbeef")
    with pytest.raises(RuntimeError, match="validated with"):
        build.require_validated_hipcc(spec)
    with pytest.raises(RuntimeError, match="validated with"):
        build.build_kernel(spec, None, "/nonexistent/never_written.hsaco".replace("/nonexistent", "/tmp"))
    monkeypatch.setenv("DECA_ALLOW_UNCHECKED_HIPCC", "1")
    build.require_validated_hipcc(spec)
