"""GPU parity of the MFMA GEMM kernel against oracle/gemm.py.

Inputs come from a seeded CPU generator and are copied to the device; every
launch goes through the C ABI.  Accuracy gate (the task's): with fp32
accumulation, max|c - ref| / max|ref| <= 1e-2 against the fp32 reference; the
reference's own check (atol = 1e-2 * sqrt(K / 1024), rtol = 2e-3, "excess" <= 1)
must hold too.  Against the checker's fp16-rounded result the kernel may differ
by one fp16 ulp where the fp32 sums differ in their last bits (the hardware's
accumulation order is not numpy's).
"""

import numpy as np
import pytest
import torch

from kernel_cases import GEMM_BF16_CASES, GEMM_CASES, GEMM_FULL
from oracle import gemm as og

pytestmark = pytest.mark.gpu

REL_GATE = 1e-2


def _run(M, N, K, cfg, a, b):
    from deca_amd.kernels.gemm_hip import build_gemm_tc, make_gemm_tc

    kern = build_gemm_tc(make_gemm_tc(M, N, K, cfg))
    ad, bd = a.cuda(), b.cuda()
    c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    kern(ad, bd, c)
    torch.cuda.synchronize()
    return c.cpu()


def _check(c, a, b, K):
    got = c.float().numpy()
    af, bf = a.float().numpy(), b.float().numpy()
    ref = og.gemm_f32(af, bf)
    assert np.isfinite(got).all(), "output holds NaN/inf (tile not written?)"
    assert og.max_rel_err(got, ref) <= REL_GATE
    assert og.excess(got, ref, K) <= 1.0
    want = og.gemm_f16_out(af, bf)
    ulp = np.maximum(np.abs(want), 2.0**-14) * 2.0**-10
    # fp32 sums of K terms differ by a few fp32 ulps between orders: that moves
    # the fp16 rounding by at most one ulp, and only near rounding boundaries
    assert np.all(np.abs(got - want) <= ulp * 1.001 + 1e-3 * np.sqrt(K / 1024) * 0.05)
    assert (got != want).mean() < 0.05


@pytest.mark.parametrize("M,N,K,cfg", GEMM_CASES, ids=lambda v: str(v))
def test_gemm_parity(M, N, K, cfg):
    from deca_amd.kernels.gemm_bench import make_inputs_cpu

    print(f"case gemm {M}x{N}x{K} {cfg}", flush=True)
    a, b = make_inputs_cpu(M, N, K, seed=M + N + K)
    _check(_run(M, N, K, cfg, a, b), a, b, K)


def test_gemm_uniform_inputs():
    """Entries ~ U(-1, 1), the distribution of the benchmark configuration."""
    from deca_amd.kernels.gemm_bench import make_inputs_cpu

    M, N, K, cfg = GEMM_CASES[0]
    a, b = make_inputs_cpu(M, N, K, seed=1, dist="uniform")
    _check(_run(M, N, K, cfg, a, b), a, b, K)


def test_gemm_closed_forms():
    """Identity, one-hot and all-ones operands pin layout and transposition."""
    M, N, K, cfg = GEMM_CASES[0]
    g = torch.Generator().manual_seed(3)
    a = torch.randn(M, K, generator=g).half()
    eye = torch.eye(K, N).half()
    assert torch.equal(_run(M, N, K, cfg, a, eye), a)           # A @ I == A
    b = torch.randn(K, N, generator=g).half()
    assert torch.equal(_run(M, N, K, cfg, torch.eye(M, K).half(), b), b)  # I @ B == B
    ones = _run(M, N, K, cfg, torch.ones(M, K).half(), torch.ones(K, N).half())
    assert torch.equal(ones, torch.full((M, N), float(K)).half())
    # one-hot row of A at column 5 picks row 5 of B, in row 3 of C only
    e = torch.zeros(M, K).half()
    e[3, 5] = 1
    c = _run(M, N, K, cfg, e, b)
    assert torch.equal(c[3], b[5]) and c[:3].abs().sum() == 0 and c[4:].abs().sum() == 0


def test_gemm_fp32_accumulation():
    """K = 2048 entries of 0.01 per output: the fp32 sum 2048 * 0.01^2 survives;
    also sums above 2048 (where fp16 cannot count by ones) stay exact."""
    M, N, K, cfg = GEMM_CASES[8]  # K = 2048
    v = torch.full((M, K), 0.01).half()
    w = torch.full((K, N), 0.01).half()
    c = _run(M, N, K, cfg, v, w).float()
    want = K * float(v[0, 0]) ** 2
    assert (c - want).abs().max() < 2e-4
    a = torch.full((M, K), 2.0).half()
    b = torch.ones(K, N).half()
    assert torch.equal(_run(M, N, K, cfg, a, b), torch.full((M, N), 4096.0).half())


@pytest.mark.parametrize("M,N,K,cfg", GEMM_FULL, ids=lambda v: str(v))
def test_gemm_full_size(M, N, K, cfg):
    """Benchmark sizes: a strided sample of rows against the CPU checker, and
    the whole result against the fp32 product computed on the device."""
    from deca_amd.kernels.gemm_bench import make_inputs_cpu
    from deca_amd.kernels.gemm_hip import build_gemm_tc, make_gemm_tc

    print(f"full-size gemm {M}x{N}x{K} {cfg}", flush=True)
    a, b = make_inputs_cpu(M, N, K, seed=0, dist="uniform")
    kern = build_gemm_tc(make_gemm_tc(M, N, K, cfg))
    ad, bd = a.cuda(), b.cuda()
    c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    kern(ad, bd, c)
    torch.cuda.synchronize()
    assert torch.isfinite(c).all()
    rows = torch.arange(0, M, M // 64)
    sub = c[rows].cpu()
    _check(sub, a[rows], b, K)
    # all rows: fp32 product on the device, row blocks to bound memory
    worst = 0.0
    scale = 0.0
    for r0 in range(0, M, 1024):
        ref = ad[r0:r0 + 1024].float() @ bd.float()
        worst = max(worst, (c[r0:r0 + 1024].float() - ref).abs().max().item())
        scale = max(scale, ref.abs().max().item())
    assert worst / scale <= REL_GATE


@pytest.mark.parametrize("M,N,K,cfg", GEMM_BF16_CASES, ids=lambda v: str(v))
def test_gemm_bf16_parity(M, N, K, cfg):
    """bf16 inputs and output, fp32 accumulation: same gate (max rel err <= 1e-2
    against the fp32 product), and at most one bf16 ulp from the checker."""
    from deca_amd.kernels.gemm_bench import make_inputs_cpu
    from deca_amd.kernels.gemm_hip import build_gemm_tc, make_gemm_tc

    print(f"case gemm bf16 {M}x{N}x{K} {cfg}", flush=True)
    a, b = make_inputs_cpu(M, N, K, seed=K, dtype=torch.bfloat16)
    kern = build_gemm_tc(make_gemm_tc(M, N, K, cfg, "bfloat16"))
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    kern(a.cuda(), b.cuda(), c)
    torch.cuda.synchronize()
    got = c.float().cpu().numpy()
    af, bf = a.float().numpy(), b.float().numpy()
    ref = og.gemm_f32(af, bf)
    assert np.isfinite(got).all()
    assert og.max_rel_err(got, ref) <= REL_GATE
    want = og.gemm_bf16_out(af, bf)
    assert np.all(np.abs(got - want) <= np.maximum(np.abs(want), 2.0**-14) * 2.0**-7 * 1.001 + 1e-3)
    assert (got != want).mean() < 0.05
    # identity: A @ I == A exactly
    eye = torch.eye(K, N).bfloat16()
    kern(a.cuda(), eye.cuda(), c)
    torch.cuda.synchronize()
    assert torch.equal(c.cpu()[:, :min(K, N)], a[:, :min(K, N)])
