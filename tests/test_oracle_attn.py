"""Pins the attention checker (oracle/attn.py) without the GPU."""

import numpy as np
import pytest
import torch

from oracle import attn as oa


def _qkv(B, H, Sq, Skv, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda S: torch.randn(B, H, S, D, generator=g).half().float().numpy()  # noqa: E731
    return mk(Sq), mk(Skv), mk(Skv)


@pytest.mark.parametrize("causal", [False, True])
def test_plain_matches_torch_composite(causal):
    q, k, v = _qkv(1, 2, 96, 96, 64)
    s = torch.from_numpy(q) @ torch.from_numpy(k).transpose(-1, -2) / 8.0
    if causal:
        s = s.masked_fill(~torch.ones(96, 96, dtype=torch.bool).tril(), float("-inf"))
    ref = (torch.softmax(s, -1) @ torch.from_numpy(v)).numpy()
    assert np.abs(oa.attention_f32(q, k, v, None, causal) - ref).max() < 2e-6


def test_constant_v_and_zero_k():
    q, k, v = _qkv(1, 1, 64, 128, 64, seed=1)
    vc = np.full_like(v, 0.375)
    for fn in (oa.attention_f32, lambda *a: oa.flash_blockwise(*a, Br=32, Bc=32)):
        assert np.abs(fn(q, k, vc, None, False) - 0.375).max() < 1e-3
    # K = 0: uniform attention -> O is the mean of V; causal: the prefix mean
    k0 = np.zeros_like(k[:, :, :64])
    v64 = v[:, :, :64]
    want = v64.mean(axis=2, keepdims=True)
    assert np.abs(oa.attention_f32(q, k0, v64, None, False) - want).max() < 1e-5
    prefix = np.cumsum(v64, axis=2) / np.arange(1, 65)[None, None, :, None]
    assert np.abs(oa.attention_f32(q, k0, v64, None, True) - prefix).max() < 1e-5
    got = oa.flash_blockwise(q, k0, v64, None, True, Br=32, Bc=16)
    assert np.abs(got - prefix).max() < 2e-3
    # the first causal row sees key 0 only
    assert np.abs(oa.attention_f32(q, k[:, :, :64], v64, None, True)[0, 0, 0] - v64[0, 0, 0]).max() < 1e-6


@pytest.mark.parametrize("causal", [False, True])
def test_blockwise_matches_plain_and_tiling_does_not_matter(causal):
    q, k, v = _qkv(1, 2, 128, 128, 64, seed=2)
    ref = oa.attention_f32(q, k, v, None, causal)
    one = oa.flash_blockwise(q, k, v, None, causal, Br=128, Bc=128)
    many = oa.flash_blockwise(q, k, v, None, causal, Br=32, Bc=32)
    assert np.abs(one - ref).max() < 2e-3
    assert np.abs(many - ref).max() < 2e-3
    assert np.abs(one - many).max() < 2e-3


def test_running_max_must_see_every_tile():
    """Looking at the row max only in every second tile has no bound to stand on: the lazy
    threshold bounds p by what the max of a tile *was seen* to be, and a tile that is not
    looked at can lie any distance above it.  On keys that grow along the sequence the
    skipped tiles push p past the fp16 range (65504) and the output is lost, while the
    every-tile recurrence with the same threshold is within the gate."""
    q, k, v = _qkv(1, 1, 64, 512, 64, seed=4)
    k = k * np.linspace(0.2, 14.0, 512, dtype=np.float32)[None, None, :, None]
    k = k.astype(np.float16).astype(np.float32)
    ref = oa.attention_f32(q, k, v, None, False)
    every = oa.flash_blockwise(q, k, v, None, False, Br=64, Bc=32, lazy_tau=8.0)
    assert np.abs(every - ref).max() < 2e-3
    with np.errstate(over="ignore", invalid="ignore"):
        second = oa.flash_blockwise(q, k, v, None, False, Br=64, Bc=32, lazy_tau=8.0, max_every=2)
    assert not np.isfinite(second).all() or np.abs(second - ref).max() > 2e-3
    # the scores of a skipped tile do exceed the stale max by more than the fp16 exponent range
    sl2 = 1.4426950408889634 / 8.0
    s = np.einsum("bhqd,bhkd->bhqk", q, k)[0, 0] * sl2
    seen = np.maximum.accumulate(s.reshape(64, 16, 32).max(-1), axis=1)
    assert (s.reshape(64, 16, 32).max(-1)[:, 1:] - seen[:, :-1]).max() > 16 + 8


@pytest.mark.parametrize("groups", [(8, 4), None])
def test_trusted_running_max_is_checked_after_the_fact(groups):
    """`FAConfig.trust`: a tile's exponentials against the running max as it stands, without
    the tile's own max.  What makes that safe is the check behind it -- a lane's p are bounded
    by their sum, and a wave whose lane sums pass 2^15 does the tile again with its max.  On
    ordinary inputs no tile is done again and the result is the eager recurrence's; on keys
    that grow along the sequence tiles are done again and the result stays within the gate;
    with the check taken away (an infinite bound) the same input pushes p past the fp16
    range and the output is lost."""
    q, k, v = _qkv(1, 2, 128, 512, 64, seed=2)
    for causal in (False, True):
        kk, vv = (k[:, :, :128], v[:, :, :128]) if causal else (k, v)
        ref = oa.attention_f32(q, kk, vv, None, causal)
        st = {}
        got = oa.flash_blockwise(q, kk, vv, None, causal, Br=64, Bc=32, lazy_tau=8.0, trust_bound=2.0 ** 15,
                                 key_groups=groups, sum_p16=groups is None, stats=st)
        assert np.abs(got - ref).max() < 2e-3
        assert st["trusted"] > 0 and st.get("redone", 0) == 0
    # growing keys: the running max is outgrown again and again
    q, k, v = _qkv(1, 1, 64, 512, 64, seed=4)
    k = k * np.linspace(0.2, 14.0, 512, dtype=np.float32)[None, None, :, None]
    k = k.astype(np.float16).astype(np.float32)
    ref = oa.attention_f32(q, k, v, None, False)
    st = {}
    with np.errstate(over="ignore", invalid="ignore"):
        checked = oa.flash_blockwise(q, k, v, None, False, Br=64, Bc=32, lazy_tau=8.0, trust_bound=2.0 ** 15,
                                     key_groups=groups, sum_p16=groups is None, stats=st)
        blind = oa.flash_blockwise(q, k, v, None, False, Br=64, Bc=32, lazy_tau=8.0, trust_bound=np.inf,
                                   key_groups=groups, sum_p16=groups is None)
    assert np.abs(checked - ref).max() < 2e-3
    assert 0 < st["redone"] < st["trusted"]
    assert not np.isfinite(blind).all() or np.abs(blind - ref).max() > 2e-3
    # the bound: while every lane sum stays within 2^15, every p does, and fp16 holds it
    assert np.float16(2.0 ** 15) == 2.0 ** 15 and np.isfinite(np.float16(2.0 ** 15))


@pytest.mark.parametrize("causal", [False, True])
def test_lazy_running_max_is_the_same_quotient(causal):
    """The kernel's lazy running max against the reference's eager one: keys grow
    along the sequence, so that rows stay below the threshold for some tiles
    (stale max, p > 1) and cross it at others."""
    q, k, v = _qkv(1, 2, 256, 256, 64, seed=4)
    k = k * np.linspace(0.2, 6.0, 256, dtype=np.float32)[None, None, :, None]
    k = k.astype(np.float16).astype(np.float32)
    ref = oa.attention_f32(q, k, v, None, causal)
    eager = oa.flash_blockwise(q, k, v, None, causal, Br=64, Bc=32)
    lazy = oa.flash_blockwise(q, k, v, None, causal, Br=64, Bc=32, lazy_tau=8.0)
    assert np.abs(eager - ref).max() < 2e-3 and np.abs(lazy - ref).max() < 2e-3
    assert np.abs(lazy - eager).max() < 2e-3
    # the two recurrences did take different paths: count the tiles that move a max
    sl2 = 1.4426950408889634 / 8.0
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * sl2
    if causal:
        s = np.where(np.arange(256)[None, :] > np.arange(256)[:, None], -np.inf, s)
    run = np.maximum.accumulate(s.reshape(1, 2, 256, 8, 32).max(-1), axis=-1)
    steps = np.diff(run, axis=-1)
    assert (steps > 0).sum() > 2 * ((steps > 8).sum() + 1)


def test_cross_attention_lengths_and_scale():
    q, k, v = _qkv(2, 1, 64, 192, 128, seed=3)
    ref = oa.attention_f32(q, k, v, 0.05, False)
    got = oa.flash_blockwise(q, k, v, 0.05, False, Br=64, Bc=64)
    assert ref.shape == (2, 1, 64, 128) and np.abs(got - ref).max() < 2e-3
    # scale matters: a different scale gives a different answer
    assert np.abs(oa.attention_f32(q, k, v, 0.5, False) - ref).max() > 1e-2


def test_flops():
    assert oa.attn_flops(4, 16, 4096, 4096, 128) == 4.0 * 4 * 16 * 4096 * 4096 * 128
    assert oa.attn_flops(4, 16, 4096, 4096, 128, True) == 2.0 * 4 * 16 * 4096 * 4096 * 128
