"""Pins the GEMM checker (oracle/gemm.py) without the GPU."""

import numpy as np
import torch

from oracle import gemm as og


def _rand(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(M, K, generator=g).half().float().numpy()


def test_brute_force_small():
    a, b = _rand(17, 33, 0), _rand(33, 9, 1)
    want = og.gemm_loops(a, b)
    assert np.allclose(og.gemm_f32(a, b), want, rtol=1e-5, atol=1e-5)
    assert np.abs(og.gemm_f64(a, b) - want).max() < 1e-4


def test_identity_and_one_hot_pin_the_layout():
    a = _rand(24, 24, 2)
    eye = np.eye(24, dtype=np.float32)
    assert np.array_equal(og.gemm_f16_out(a, eye), a)
    assert np.array_equal(og.gemm_f16_out(eye, a), a)
    # one-hot row of A picks a row of B; one-hot column of B picks a column of A
    b = _rand(24, 40, 3)
    e = np.zeros((1, 24), np.float32)
    e[0, 5] = 1
    assert np.array_equal(og.gemm_f16_out(e, b)[0], b[5])
    f = np.zeros((24, 1), np.float32)
    f[7, 0] = 1
    assert np.array_equal(og.gemm_f16_out(a, f)[:, 0], a[:, 7])
    # A @ B != B^T-style products: a non-symmetric case
    a2 = np.arange(6, dtype=np.float32).reshape(2, 3)
    b2 = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal(og.gemm_f16_out(a2, b2), np.array([[20, 23, 26, 29], [56, 68, 80, 92]], np.float32))


def test_all_ones_counts_k():
    for K in (64, 2048):
        c = og.gemm_f16_out(np.ones((8, K), np.float32), np.ones((K, 8), np.float32))
        assert np.array_equal(c, np.full((8, 8), K, np.float32))


def test_fp32_accumulation_discriminator():
    """K = 16384 entries of fp16(0.01): the fp32 sum is 16384 * 0.01^2 = 1.64;
    an fp16 accumulator would stall far below it."""
    K = 16384
    v = np.float32(np.float16(0.01))
    c = og.gemm_f16_out(np.full((2, K), v, np.float32), np.full((K, 2), v, np.float32))
    assert abs(c[0, 0] - K * float(v) ** 2) < 2e-3


def test_error_metrics():
    ref = np.array([[1.0, -2.0], [0.0, 4.0]], np.float32)
    c = ref + np.array([[0.001, 0.0], [0.0, -0.004]], np.float32)
    assert abs(og.max_rel_err(c, ref) - 0.001) < 1e-6
    atol, rtol = og.tolerance(1024)
    assert atol == 1e-2 and rtol == 2e-3
    assert abs(og.excess(c, ref, 1024) - 0.004 / (1e-2 + 2e-3 * 4)) < 1e-4
    assert og.gemm_flops(8192, 8192, 8192) == 2.0 * 8192**3


def test_bf16_output_rounding():
    a, b = _rand(16, 64, 4), _rand(64, 16, 5)
    want = torch.from_numpy(og.gemm_f32(a, b)).bfloat16().float().numpy()
    assert np.array_equal(og.gemm_bf16_out(a, b), want)
