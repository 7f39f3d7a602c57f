"""Configurations the solvers emit for a few small shapes, run once on the GPU against
torch's fp32 result of the same operator.

By default an evenly spaced sample of each solver's list runs (SAMPLE configurations per
shape; `kernel_cases.all_specs()` names the same kernels, so the build step compiles them
beforehand).  With DECA_ALL_CONFIGS=1 every configuration runs (every GEMM_STRIDE-th for the
GEMM): several thousand code objects, minutes of host time to compile.  Gates are the ones of
the other GPU tests.
"""

import os
from concurrent.futures import ThreadPoolExecutor

import pytest
import torch

from kernel_cases import (SOLVER_FA_SHAPES as FA_SHAPES, SOLVER_GEMM_SHAPES as GEMM_SHAPES,
                          SOLVER_ROW_SHAPES as ROW_SHAPES, solver_sample)

pytestmark = [pytest.mark.gpu]

EVERY = os.environ.get("DECA_ALL_CONFIGS") == "1"
GEMM_STRIDE = int(os.environ.get("DECA_ALL_CONFIGS_GEMM_STRIDE", "7"))  # 1: every GEMM config
GEMM_MFMA = os.environ.get("DECA_ALL_CONFIGS_GEMM_MFMA")  # "16" / "32": only that MFMA tile form
GEMM_AGPR = os.environ.get("DECA_ALL_CONFIGS_GEMM_AGPR")  # "1" / "0": only configs with / without agpr
FA_TRUST = os.environ.get("DECA_ALL_CONFIGS_FA_TRUST")  # "1" / "0": only attention configs with / without trust


def gemm_configs(M, N, K):
    from deca_amd import Solver

    configs = Solver.solve_gemm_tc(_arch(), M, N, K)
    if not EVERY:
        return solver_sample(configs)
    if GEMM_MFMA:
        configs = [c for c in configs if c.mfma == int(GEMM_MFMA)]
    if GEMM_AGPR:
        configs = [c for c in configs if c.agpr == (GEMM_AGPR == "1")]
    return configs[::GEMM_STRIDE]


def _build_all(specs):
    """Paths of the code objects; None where the build step refused the generated code
    (`build.check_generated_code`), as the tuner drops such a config."""
    from deca_amd.kernels.build import cached_build

    def one(spec):
        try:
            return cached_build(spec)
        except RuntimeError as err:
            if "accumulation-register moves" not in str(err):
                raise
            print(f"refused {err}", flush=True)
            return None

    with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as pool:
        return list(pool.map(one, specs))


def _launch(what, kern, *args):
    """One launch, named on stdout before it starts; a HIP error ends the whole session (the
    device is not to be used after a fault), a wrong result is only collected by the caller."""
    print(f"launch {what}", flush=True)
    try:
        kern(*args)
        torch.cuda.synchronize()
    except RuntimeError as err:
        pytest.exit(f"HIP error in {what}: {err}", returncode=3)


def _report(wrong):
    """Every wrong configuration on stdout (an assertion message is cut short)."""
    for name, err in wrong:
        print(f"WRONG {name}: {err:.3e}", flush=True)


MIN_LAUNCHED = 0.9


def _load(spec, path, tally):
    """The loaded kernel, or None for a config the tuner would drop as well: one whose
    generated code the build step refused (`path is None`: only kernels that make promises
    about their code can be), or whose code object the loader rejects (only kernels marked
    `no_scratch`, when they spill).  Both are counted."""
    from deca_amd.driver.driver import KernelRejected, load_kernel

    meta = dict(spec.meta)
    if path is None:
        assert "accumulator_moves" in meta, f"an unchecked build was refused: {meta.get('cfg')}"
        tally["refused"] += 1
        return None
    try:
        kern = load_kernel(spec, path)
    except KernelRejected as err:
        assert meta.get("no_scratch"), f"rejected without the mark: {err}"
        print(f"rejected {err}", flush=True)
        tally["rejected"] += 1
        return None
    tally["launched"] += 1
    return kern


def _coverage(what, tally, total):
    """What ran and what did not, on stdout; the sample must not shrink unnoticed."""
    print(f"coverage {what}: {tally['launched']} launched, {tally['refused']} refused by the build "
          f"step, {tally['rejected']} rejected by the loader, of {total}", flush=True)
    assert sum(tally.values()) == total
    assert tally["launched"] >= MIN_LAUNCHED * total, (what, tally)


def _arch():
    from deca_amd.arch.MI355X import MI355X

    return MI355X()


@pytest.mark.parametrize("B,H,S,D,causal", FA_SHAPES)
def test_every_flash_attn_config(B, H, S, D, causal):
    from deca_amd import Solver
    from deca_amd.kernels.attn_bench import make_qkv, math_attention
    from deca_amd.kernels.flash_attn_hip import make_flash_attn_fwd

    configs = Solver.solve_flash_attn(_arch(), B, H, S, S, D)
    if not EVERY:
        configs = solver_sample(configs)
    elif FA_TRUST:
        configs = [c for c in configs if c.trust == (FA_TRUST == "1")]
    specs = [make_flash_attn_fwd(B, H, S, S, D, cfg, None, causal) for cfg in configs]
    paths = _build_all(specs)
    q, k, v = make_qkv(B, H, S, S, D)
    ref = math_attention(q, k, v, causal)
    wrong, tally = [], {"launched": 0, "refused": 0, "rejected": 0}
    for cfg, spec, path in zip(configs, specs, paths):
        kern = _load(spec, path, tally)
        if kern is None:
            continue
        o = torch.full_like(q, float("nan"))
        _launch(f"fa B{B} H{H} S{S} D{D} causal={causal} {cfg}", kern, q, k, v, o)
        err = (o.float() - ref).abs().max().item()
        if not err <= 2e-3:
            wrong.append((str(cfg), err))
    _report(wrong)
    _coverage(f"fa B{B} H{H} S{S} D{D} causal={causal}", tally, len(configs))
    assert not wrong, wrong[:8]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_every_gemm_config(M, N, K):
    from deca_amd.kernels.gemm_bench import make_inputs
    from deca_amd.kernels.gemm_hip import make_gemm_tc

    configs = gemm_configs(M, N, K)
    specs = [make_gemm_tc(M, N, K, cfg) for cfg in configs]
    paths = _build_all(specs)
    a, b = make_inputs(M, N, K)
    ref = a.float() @ b.float()
    scale = ref.abs().max().item()
    wrong, tally = [], {"launched": 0, "refused": 0, "rejected": 0}
    for cfg, spec, path in zip(configs, specs, paths):
        kern = _load(spec, path, tally)
        if kern is None:
            continue
        c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        _launch(f"gemm {M}x{N}x{K} {cfg}", kern, a, b, c)
        err = (c.float() - ref).abs().max().item() / scale
        if not err <= 1e-2:
            wrong.append((str(cfg), err))
    _report(wrong)
    _coverage(f"gemm {M}x{N}x{K}", tally, len(configs))
    assert not wrong, wrong[:8]


@pytest.mark.parametrize("op,M,N,dtype", ROW_SHAPES)
def test_every_rowwise_config(op, M, N, dtype):
    from deca_amd import Solver
    from deca_amd.driver.driver import load_kernel
    from deca_amd.kernels.rowwise_bench import make_inputs
    from deca_amd.kernels.rowwise_hip import make_rowwise

    configs = Solver.solve_rowwise(_arch(), op, M, N)
    if not EVERY:
        configs = solver_sample(configs)
    specs = [make_rowwise(op, M, N, dtype, cfg, 1e-6) for cfg in configs]
    paths = _build_all(specs)
    inputs = make_inputs(op, M, N, dtype, std=2.0 if op == "softmax" else 1.0)
    x = inputs[0].float()
    if op == "softmax":
        ref = torch.softmax(x, -1)
    else:
        normed = (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6)).to(inputs[0].dtype).float()
        ref = normed * inputs[1].float()
    tol = 1e-2 if dtype == "bfloat16" else 2e-3
    wrong = []
    for cfg, spec, path in zip(configs, specs, paths):
        y = torch.full_like(inputs[0], float("nan"))
        _launch(f"{op} {dtype} {M}x{N} {cfg}", load_kernel(spec, path), *inputs, y)
        err = ((y.float() - ref).abs() / ref.abs().clamp(min=1.0)).max().item()
        if not err <= tol:
            wrong.append((str(cfg), err))
    _report(wrong)
    assert not wrong, wrong[:8]
