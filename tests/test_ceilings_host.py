"""Host checks of the ceilings probe: its specialisations are distinct code objects and
compile for gfx950 without spilling (the GPU side is a measurement, not a test)."""

from deca_amd.arch import ceilings
from deca_amd.kernels.build import kernel_resources


def test_probe_specs_cover_every_family_once():
    specs = ceilings.all_specs()
    modes = {dict(s.defines)["DECA_CEILING"] for s in specs}
    assert modes == {0, 1, 2, 3, 4, 5, 6}
    # grids differ between some variants; every (macros, options) set names one code object
    keyed = {}
    for s in specs:
        keyed.setdefault(s.key(), set()).add(tuple(sorted(dict(s.defines).items())))
    assert all(len(v) == 1 for v in keyed.values())


def test_probe_kernels_compile_without_spills():
    picks = [ceilings.lds_spec(4, 4), ceilings.valu_spec(7, 1), ceilings.valu_spec(13, 0, 1),
             ceilings.mfma_spec(4, 16, 1024)]
    for spec in picks:
        res = kernel_resources(spec)
        assert res.get("vgpr_spills", 0) == 0 and res.get("scratch_bytes", 0) == 0, (spec.show(), res)
    # the accumulation-register variant really keeps its accumulators there
    assert kernel_resources(ceilings.valu_spec(7, 1)).get("agprs", 0) >= 64
