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
