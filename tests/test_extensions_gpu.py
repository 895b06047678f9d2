"""GPU tests of what goes beyond the reference's kernel but is declared in its parameter block (reference
csrc/flash.h:36-45,56): grouped-query attention, the log-sum-exp output and causal masks for seqlen_q != seqlen_k.
Same gate as the parity tests (oracle/parity_gate.py): strict max-abs <= 2e-2 and mean-abs <= 2e-3 against the oracle in the
device's arithmetic; the log-sum-exp to 5e-6 relative (the logits are emulated exactly; the row sum is an fp32 sum in
another order and the device's exp2 and log2 are accurate to an ulp)."""
import math

import numpy as np
import pytest
import torch

import cutlass_flash_atten_fp8_amd as fa
from oracle import fa8_oracle as fo  # noqa: F401
from oracle.parity_gate import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LSE_TOL = 5e-6        # against the oracle in the device's arithmetic
EXACT_LSE_TOL = 5e-4  # against an exact fp64 log-sum-exp: the matrix instruction cuts products 13 bits below their group's largest


def rand_fp8(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.float8_e4m3fn)


def u8(t):
    return t.view(torch.uint8).cpu().numpy()


def gate(o, lse, q, k, v, scale, causal, bottom_right=False, label=""):
    got = o.float().cpu().numpy()
    _, ref_lse = assert_parity(got, u8(q), u8(k), u8(v), scale, causal=causal, kv_block=fa.query(fa.FA8_QUERY_KV_BLOCK),
                               causal_bottom_right=bottom_right, label="ext " + label)
    if lse is not None:
        got_lse = lse.cpu().numpy()
        empty = np.isneginf(ref_lse)
        assert np.array_equal(np.isneginf(got_lse), empty), label
        assert np.abs(got_lse[~empty] - ref_lse[~empty]).max() <= LSE_TOL * max(1.0, np.abs(ref_lse[~empty]).max()), label
        assert (got[empty] == 0).all(), label  # a query that sees no key: all-zero row


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("h,hk,d", [(8, 2, 128), (8, 1, 64), (6, 3, 256), (16, 4, 96)])
def test_grouped_query_attention(h, hk, d, causal):
    q = rand_fp8((2, h, 300, d), 1)
    k, v = rand_fp8((2, hk, 300, d), 2), rand_fp8((2, hk, 300, d), 3)
    scale = 1 / math.sqrt(d)
    o, lse = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale, return_lse=True)
    gate(o, lse, q, k, v, scale, causal, label=f"gqa h={h} hk={hk} d={d} causal={causal}")
    # the same arithmetic as multi-head attention on repeated k/v heads: bitwise equal
    rep = h // hk
    k_rep = k.view(torch.uint8).repeat_interleave(rep, dim=1).view(torch.float8_e4m3fn)
    v_rep = v.view(torch.uint8).repeat_interleave(rep, dim=1).view(torch.float8_e4m3fn)
    o2, lse2 = fa.flash_attention_v2_cutlass(q.to(DEV), k_rep.to(DEV), v_rep.to(DEV), causal, scale, return_lse=True)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)


def test_grouped_query_attention_through_the_binding_and_transposed_v():
    ext = fa.load_extension()
    q = rand_fp8((2, 8, 208, 128), 4).to(DEV)
    k, v = rand_fp8((2, 2, 208, 128), 5).to(DEV), rand_fp8((2, 2, 208, 128), 6).to(DEV)
    o, lse = ext.flash_attention_v2_cutlass(q, k, v, True, 0.09, return_lse=True)
    o_m, lse_m = fa.flash_attention_v2_cutlass(q, k, v, True, 0.09, return_lse=True)
    ot = ext.flash_attention_v2_cutlass(q, k, v.transpose(2, 3).contiguous(), True, 0.09, v_transposed=True)
    assert len(ot) == 1
    torch.cuda.synchronize()
    assert torch.equal(o, o_m) and torch.equal(lse, lse_m) and torch.equal(o, ot[0])
    assert lse.dtype == torch.float32 and tuple(lse.shape) == (2, 8, 208)
    with pytest.raises(RuntimeError, match="multiple"):
        ext.flash_attention_v2_cutlass(q, k[:, :1].repeat(1, 3, 1, 1), v[:, :1].repeat(1, 3, 1, 1), False, 0.09)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("n,d", [(1, 64), (100, 32), (129, 128), (1000, 128), (333, 224)])
def test_log_sum_exp(n, d, causal):
    q, k, v = (rand_fp8((2, 3, n, d), s, 1.5) for s in (7, 8, 9))
    scale = 1 / math.sqrt(d)
    o, lse = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale, return_lse=True)
    o_plain = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale)[0]
    assert torch.equal(o, o_plain)  # asking for the log-sum-exp does not change O
    gate(o, lse, q, k, v, scale, causal, label=f"lse n={n} d={d} causal={causal}")
    # and against a direct fp64 logsumexp of the scaled logits
    s = torch.einsum("bhid,bhjd->bhij", q.double(), k.double()) * scale
    if causal:
        s = s.masked_fill(~torch.ones(n, n, dtype=torch.bool).tril(), -math.inf)
    want = torch.logsumexp(s, dim=-1).numpy()
    assert np.abs(lse.cpu().numpy() - want).max() <= EXACT_LSE_TOL * max(1.0, np.abs(want).max())


def test_log_sum_exp_merges_a_kv_split():
    """The use the output is for: attention over [K1;K2] from two runs over K1 and K2, merged with their log-sum-exps."""
    q = rand_fp8((1, 4, 256, 128), 10)
    k, v = rand_fp8((1, 4, 512, 128), 11), rand_fp8((1, 4, 512, 128), 12)
    scale = 1 / math.sqrt(128)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    full, lse = fa.flash_attention_v2_cutlass(qd, kd, vd, False, scale, return_lse=True)
    o1, l1 = fa.flash_attention_v2_cutlass(qd, kd[:, :, :256].contiguous(), vd[:, :, :256].contiguous(), False, scale, return_lse=True)
    o2, l2 = fa.flash_attention_v2_cutlass(qd, kd[:, :, 256:].contiguous(), vd[:, :, 256:].contiguous(), False, scale, return_lse=True)
    l12 = torch.logaddexp(l1, l2)
    merged = o1.float() * torch.exp(l1 - l12)[..., None] + o2.float() * torch.exp(l2 - l12)[..., None]
    assert (l12 - lse).abs().max() <= EXACT_LSE_TOL
    # the two halves quantise P against their own running max: equal to the one-pass result within the parity tolerance
    assert (merged - full.float()).abs().max() <= 2e-2 and (merged - full.float()).abs().mean() <= 2e-3


@pytest.mark.parametrize("bottom_right", [False, True])
@pytest.mark.parametrize("nq,nk,d", [(40, 200, 128), (200, 40, 128), (130, 131, 64), (1, 500, 128), (500, 1, 64), (300, 1000, 128),
                                     (1000, 300, 256), (128, 192, 32)])
def test_causal_with_different_lengths(nq, nk, d, bottom_right):
    q = rand_fp8((2, 2, nq, d), 13)
    k, v = rand_fp8((2, 2, nk, d), 14), rand_fp8((2, 2, nk, d), 15)
    scale = 1 / math.sqrt(d)
    o, lse = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, scale, return_lse=True,
                                           causal_bottom_right=bottom_right)
    gate(o, lse, q, k, v, scale, True, bottom_right, label=f"causal nq={nq} nk={nk} d={d} bottom_right={bottom_right}")
    if not bottom_right and nq <= nk:
        # top-left: the keys past the last query are never seen, so the result equals the square problem on the first nq keys
        sq = fa.flash_attention_v2_cutlass(q.to(DEV), k[:, :, :nq].contiguous().to(DEV), v[:, :, :nq].contiguous().to(DEV), True, scale)[0]
        assert torch.equal(o, sq)
