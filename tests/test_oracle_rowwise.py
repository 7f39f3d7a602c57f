"""Pins the row-wise checker (oracle/rowwise.py) without the GPU: library
routines on the CPU, closed forms and invariants chosen so that a dropped
term, a wrong neutral value or a misplaced rounding fails at least one."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import rowwise as orw


def _randn(M, N, dtype, seed=0, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (std * torch.randn(M, N, generator=g)).to(dtype)


def test_bf16_rounding_matches_torch():
    g = torch.Generator().manual_seed(1)
    a = torch.randn(200000, generator=g) * 37.0
    a[:4] = torch.tensor([0.0, -0.0, 3.0e38, -3.0e38])
    got = orw.round_to_dtype(a.numpy(), "bfloat16")
    assert np.array_equal(got, a.bfloat16().float().numpy())
    # ties go to even: 1 + 2^-8 is halfway between bf16 neighbours 1 and 1 + 2^-7
    tie = np.array([1.0 + 2.0**-8, 1.0 + 2.0**-7 + 2.0**-8], np.float32)
    assert np.array_equal(orw.round_to_dtype(tie, "bfloat16"),
                          np.array([1.0, 1.0 + 2.0**-6], np.float32))


@pytest.mark.parametrize("dtype,tdt,tol", [("float16", torch.float16, 1e-6), ("bfloat16", torch.bfloat16, 1e-6)])
def test_softmax_matches_torch(dtype, tdt, tol):
    x = _randn(96, 4096, tdt, std=2.0)
    ref = torch.softmax(x.float(), -1)  # fp32 library routine
    got = orw.softmax_reg(orw.to_f32(x), dtype)
    # same value up to the final rounding to `dtype`
    want = orw.round_to_dtype(ref.numpy(), dtype)
    ulp = np.maximum(np.abs(want), 1e-30) * (2.0**-10 if dtype == "float16" else 2.0**-7)
    assert np.all(np.abs(got - want) <= ulp + tol)
    assert (got != want).mean() < 2e-3  # only double-rounding ties may differ


def test_softmax_invariants():
    x = orw.to_f32(_randn(32, 1000, torch.float16, seed=3, std=3.0))
    y = orw.softmax_reg(x, "float16")
    assert np.allclose(y.sum(-1), 1.0, atol=1000 * 2.0**-12)
    # shift invariance (exactly representable shift keeps fp16 inputs exact)
    y2 = orw.softmax_reg(x + np.float32(8.0), "float16")
    assert np.abs(y - y2).max() <= 2.0**-11
    # constant row -> 1/N exactly after rounding
    c = np.full((2, 512), 3.25, np.float32)
    assert np.array_equal(orw.softmax_reg(c, "float16"),
                          np.full((2, 512), np.float32(np.float16(1.0 / 512)), np.float32))
    # one dominant entry -> one-hot; fp16 max must not overflow
    d = np.zeros((1, 64), np.float32)
    d[0, 5] = 65504.0
    out = orw.softmax_reg(d, "float16")
    assert out[0, 5] == 1.0 and out.sum() == 1.0 and np.isfinite(out).all()
    # ordering is preserved
    assert np.array_equal(np.argsort(x[0], kind="stable")[-5:], np.argsort(y[0] + x[0] * 1e-12, kind="stable")[-5:])


@pytest.mark.parametrize("N,tpr,vec,unroll", [(4096, 128, 8, 2), (4000, 128, 8, 2), (1000, 64, 4, 1),
                                               (32000, 1024, 8, 4), (640, 16, 8, 4)])
def test_softmax_twopass_equals_reg(N, tpr, vec, unroll):
    x = orw.to_f32(_randn(8, N, torch.float16, seed=N, std=2.0))
    a = orw.softmax_reg(x, "float16")
    b = orw.softmax_twopass(x, "float16", tpr, vec, unroll)
    # different summation order: equal up to one fp16 ulp of the largest outputs
    assert np.abs(a - b).max() <= 2.0**-11 * max(a.max(), 2.0**-14) * 2 + 1e-9


@pytest.mark.parametrize("dtype,tdt", [("float16", torch.float16), ("bfloat16", torch.bfloat16)])
def test_rmsnorm_matches_torch_composite(dtype, tdt):
    """The reference rounds x * r to the I/O dtype before the weight multiply
    (rowwise_tir.py:340-344); that is torch's eager composite in `dtype`."""
    x = _randn(64, 4096, tdt, seed=5)
    g = torch.Generator().manual_seed(6)
    w = (1.0 + 0.1 * torch.randn(4096, generator=g)).to(tdt)
    got = orw.rmsnorm(orw.to_f32(x), orw.to_f32(w), 1e-6, dtype)
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)
    comp = ((xf * r).to(tdt) * w).float().numpy()
    assert (got != comp).mean() < 1e-3
    eps_rel = 2.0**-10 if dtype == "float16" else 2.0**-7
    assert np.all(np.abs(got - comp) <= np.abs(comp) * eps_rel + 1e-12)
    # and the fused library routine (one rounding) agrees up to the extra
    # rounding, whose half-ulp can weigh up to 1.4 ulp of a smaller product
    lib = F.rms_norm(x, (4096,), w, eps=1e-6).float().numpy()
    assert np.all(np.abs(got - lib) <= 2 * np.abs(lib) * eps_rel + 1e-12)


def test_rmsnorm_closed_forms():
    eps = 1e-6
    ones = np.ones((3, 256), np.float32)
    want = np.float32(np.float16(1.0 / np.sqrt(1.0 + eps)))
    assert np.array_equal(orw.rmsnorm(ones, ones[0], eps, "float16"), np.full((3, 256), want))
    # scale invariance: x -> 4x leaves y unchanged (up to eps, far below fp16 resolution)
    g = torch.Generator().manual_seed(9)
    x = orw.to_f32(torch.randn(16, 512, generator=g).half())
    w = orw.to_f32((1 + 0.1 * torch.randn(512, generator=g)).half())
    a = orw.rmsnorm(x, w, eps, "float16")
    b = orw.rmsnorm(4 * x, w, eps, "float16")
    assert (a != b).mean() < 5e-3
    # weight is applied per column: doubling one weight doubles that column only
    w2 = w.copy()
    w2[7] *= 2
    c = orw.rmsnorm(x, w2, eps, "float16")
    assert np.array_equal(c[:, 7], 2 * a[:, 7]) and np.array_equal(np.delete(c, 7, 1), np.delete(a, 7, 1))
    # mean of squares of the normalised row is ~1
    n = orw.rmsnorm(x, np.ones(512, np.float32), eps, "float16")
    assert np.allclose((n * n).mean(-1), 1.0, atol=2e-3)
    # eps matters when the row is tiny: x = 1e-3 everywhere, eps = 1e-6 -> 1/sqrt(2)
    tiny = np.full((1, 64), 1e-3, np.float32)
    got = orw.rmsnorm(orw.round_to_dtype(tiny, "float16"), np.ones(64, np.float32), 1e-6, "float16")
    assert abs(got[0, 0] - 1 / np.sqrt(2)) < 2e-3


def test_rowwise_bytes():
    assert orw.rowwise_bytes("softmax", 16384, 4096) == 268435456
    assert orw.rowwise_bytes("rmsnorm", 16384, 4096) == 268443648
    assert orw.rowwise_bytes("rmsnorm", 8192, 8192) == 268451840
