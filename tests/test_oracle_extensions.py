"""Pins the oracle's extensions beyond the reference (oracle/fa8_oracle.c: heads_k, causal_shift, lse) by what the
mathematics fixes: grouped-query attention equals multi-head attention on repeated k/v heads, the log-sum-exp equals a
direct fp64 logsumexp of the scaled logits, and a shifted causal mask equals a brute-force boolean mask.
"""
import numpy as np
import pytest

from oracle import fa8_oracle as fo
from oracle import np_restatement as nr


def enc(x):
    return nr.encode_rne_sat(np.asarray(x, dtype=np.float64))


def dec(c):
    return nr.decode(c)


def rand(rng, shape, s=1.0):
    return enc(rng.standard_normal(shape) * s)


def masked_logits(q, k, scale, causal, shift):
    """fp64 scaled logits [B,H,Nq,Nk] with -inf where column j > row i + shift (k already expanded to q's heads)."""
    s = np.einsum("bhid,bhjd->bhij", dec(q), dec(k)) * scale
    if causal:
        i = np.arange(q.shape[2])[:, None]
        j = np.arange(k.shape[2])[None, :]
        s = np.where(j <= i + shift, s, -np.inf)
    return s


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("hk", [1, 2, 6])
def test_grouped_query_equals_repeated_heads(hk, causal):
    rng = np.random.default_rng(50 + hk)
    q = rand(rng, (2, 6, 150, 64))
    k, v = rand(rng, (2, hk, 150, 64)), rand(rng, (2, hk, 150, 64))
    rep = 6 // hk
    got, lse = fo.forward(q, k, v, 0.125, causal=causal, out_dtype=fo.OUT_F32, return_lse=True)
    want, lse_want = fo.forward(q, np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1), 0.125, causal=causal,
                                out_dtype=fo.OUT_F32, return_lse=True)
    assert np.array_equal(got, want) and np.array_equal(lse, lse_want)
    # q head h must read k/v head h // rep, not h % hk
    if 1 < hk < 6:
        wrong = fo.forward(q, np.tile(k, (1, rep, 1, 1)), np.tile(v, (1, rep, 1, 1)), 0.125, causal=causal, out_dtype=fo.OUT_F32)
        assert not np.array_equal(got, wrong)
    f64 = fo.attention_f64(q, k, v, 0.125, causal=causal)
    assert np.array_equal(f64, fo.attention_f64(q, np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1), 0.125, causal=causal))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bc", [16, 64, 1000])
def test_lse_equals_fp64_logsumexp(bc, causal):
    rng = np.random.default_rng(60)
    q, k, v = (rand(rng, (2, 2, 200, 64), 1.5) for _ in range(3))
    scale = 0.2
    _, lse = fo.forward(q, k, v, scale, causal=causal, kv_block=bc, return_lse=True)
    s = masked_logits(q, k, scale, causal, 0)
    mx = s.max(axis=-1, keepdims=True)
    want = (mx + np.log(np.exp(s - mx).sum(axis=-1, keepdims=True)))[..., 0]
    assert np.abs(lse - want).max() < 2e-5 * max(1.0, np.abs(want).max())
    # natural log, scaled logits: scale = 0 gives log(number of visible keys)
    _, lse0 = fo.forward(q, k, v, 0.0, causal=causal, kv_block=bc, return_lse=True)
    n_vis = np.arange(1, 201) if causal else np.full(200, 200)
    assert np.abs(lse0 - np.log(n_vis)[None, None, :]).max() < 1e-5


@pytest.mark.parametrize("nq,nk", [(40, 200), (200, 40), (130, 131), (64, 64)])
@pytest.mark.parametrize("bottom_right", [False, True])
def test_causal_alignment_equals_brute_force_mask(nq, nk, bottom_right):
    rng = np.random.default_rng(70 + nq)
    q = rand(rng, (1, 2, nq, 64))
    k, v = rand(rng, (1, 2, nk, 64)), rand(rng, (1, 2, nk, 64))
    shift = nk - nq if bottom_right else 0
    s = masked_logits(q, k, 0.125, True, shift)
    visible = np.isfinite(s).any(axis=-1)  # rows that see at least one key
    with np.errstate(invalid="ignore"):
        mx = np.where(visible, s.max(axis=-1), 0.0)[..., None]
        p = np.exp(s - mx)
        den = p.sum(axis=-1, keepdims=True)
        want = np.einsum("bhij,bhjd->bhid", np.where(den > 0, p / np.where(den > 0, den, 1.0), 0.0), dec(v))
        want_lse = np.where(visible, mx[..., 0] + np.log(np.where(den[..., 0] > 0, den[..., 0], 1.0)), -np.inf)
    got, lse = fo.forward(q, k, v, 0.125, causal=True, causal_bottom_right=bottom_right, quantize_p=False,
                          out_dtype=fo.OUT_F32, return_lse=True)
    assert np.abs(got - want).max() < 5e-6
    assert np.array_equal(np.isneginf(lse), ~visible)
    assert np.abs(lse[visible] - want_lse[visible]).max() < 1e-5
    assert (got[~visible] == 0).all()  # a query that sees no key gives an all-zero row
    f64 = fo.attention_f64(q, k, v, 0.125, causal=True, causal_bottom_right=bottom_right)
    assert np.abs(f64[visible] - want[visible]).max() < 1e-12
    if nq == nk:
        assert np.array_equal(got, fo.forward(q, k, v, 0.125, causal=True, quantize_p=False, out_dtype=fo.OUT_F32))
