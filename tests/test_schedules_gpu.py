"""The three main loops of the kernel (FA8_SCHEDULE_ROLLING / _PIPELINED / _DENSE, include/fa8_api.h) perform the same
arithmetic in the same order: their outputs must be bitwise equal, for every feature of the operator.  The parity of the
result itself is the business of the parity tests; they reach the dense loop through the library's own choice (full
attention over whole KV blocks), the pipelined loop through small masked launches and the rolling loop through the large
causal configurations.  A dense hint that does not apply (causal, ragged seqlen_k) is answered with the automatic choice,
so asking for it is always valid."""
import numpy as np
import pytest
import torch

import cutlass_flash_atten_fp8_amd as fa
from oracle.parity_gate import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(seed, B, H, Hk, Nq, Nk, d, dtype, heavy=False):
    g = torch.Generator().manual_seed(seed)
    mk = (lambda *s: torch.randn(*s, generator=g) * (3.0 if heavy else 1.0))
    q, k, v = mk(B, H, Nq, d), mk(B, Hk, Nk, d), mk(B, Hk, Nk, d)
    return tuple(t.to(dtype) for t in (q, k, v))


CASES = [
    # B, H, Hk, Nq, Nk, d, causal, bottom_right, vt, in dtype, out dtype
    (1, 2, 2, 64, 64, 128, False, False, False, torch.float8_e4m3fn, torch.float16),     # a single block
    (1, 2, 2, 1, 64, 64, False, False, False, torch.float8_e4m3fn, torch.float16),       # one query, one block
    (1, 2, 2, 77, 128, 128, False, False, False, torch.float8_e4m3fn, torch.float16),    # 2 blocks, ragged queries
    (1, 2, 1, 200, 256, 64, False, False, True, torch.float8_e4m3fn, torch.float8_e4m3fn),  # 4 blocks, v^T, fp8 out, grouped
    (1, 2, 2, 300, 448, 128, False, False, True, torch.float8_e5m2, torch.float8_e5m2),  # 7 blocks
    (1, 2, 2, 65, 65, 128, True, False, False, torch.float8_e4m3fn, torch.float16),      # one row into the second block
    (2, 3, 3, 128, 128, 64, True, False, False, torch.float8_e4m3fn, torch.float16),
    (1, 2, 2, 192, 192, 128, False, False, False, torch.float8_e4m3fn, torch.float16),   # 3 blocks
    (1, 2, 2, 256, 256, 64, True, False, False, torch.float8_e4m3fn, torch.float16),     # 4
    (1, 2, 1, 320, 320, 128, True, False, False, torch.float8_e4m3fn, torch.float16),    # 5, two q heads per k/v head
    (1, 1, 1, 333, 333, 128, False, False, False, torch.float8_e4m3fn, torch.float16),   # ragged
    (1, 2, 2, 333, 333, 64, True, False, False, torch.float8_e5m2, torch.float16),
    (1, 2, 2, 1000, 1000, 128, True, False, False, torch.float8_e4m3fn, torch.float16),
    (2, 4, 2, 777, 777, 64, False, False, False, torch.float8_e4m3fn, torch.float8_e4m3fn),
    (1, 2, 2, 512, 512, 128, True, False, True, torch.float8_e4m3fn, torch.float16),     # v as [B,H,d,N]
    (1, 2, 2, 400, 400, 64, False, False, True, torch.float8_e5m2, torch.float8_e5m2),
    (1, 2, 2, 100, 700, 128, True, True, False, torch.float8_e4m3fn, torch.float16),     # decode-like, diagonal at the end
    (1, 2, 2, 700, 100, 128, True, True, False, torch.float8_e4m3fn, torch.float16),     # queries that see no key
    (1, 2, 2, 700, 100, 64, True, False, False, torch.float8_e4m3fn, torch.float16),
    (1, 3, 3, 130, 1500, 128, False, False, False, torch.float8_e4m3fn, torch.float16),
    (1, 2, 2, 2048, 2048, 128, True, False, False, torch.float8_e4m3fn, torch.float16),
    (1, 8, 8, 1024, 1024, 64, False, False, False, torch.float8_e4m3fn, torch.float16),
    (2, 32, 32, 4096, 4096, 128, False, False, False, torch.float8_e4m3fn, torch.float16),  # the headline shape
    (1, 8, 8, 8192, 8192, 128, True, False, False, torch.float8_e4m3fn, torch.float16),
    (1, 16, 4, 4160, 4160, 64, True, False, False, torch.float8_e4m3fn, torch.float16),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"B{c[0]}H{c[1]}k{c[2]}Nq{c[3]}Nk{c[4]}d{c[5]}{'c' if c[6] else 'f'}{'br' if c[7] else ''}{'vt' if c[8] else ''}")
def test_the_loops_agree_bitwise(case):
    B, H, Hk, Nq, Nk, d, causal, br, vt, in_dt, out_dt = case
    if vt and Nk % 16:
        pytest.skip("transposed v needs seqlen_k % 16 == 0")
    q, k, v = _inputs(hash(case[:7]) % 1000, B, H, Hk, Nq, Nk, d, in_dt, heavy=(Nq % 2 == 1))
    v_arg = v.transpose(2, 3).contiguous() if vt else v
    outs = {}
    for name, sched in (("rolling", fa.FA8_SCHEDULE_ROLLING), ("pipelined", fa.FA8_SCHEDULE_PIPELINED), ("dense", fa.FA8_SCHEDULE_DENSE)):
        o, lse = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v_arg.to(DEV), causal, d ** -0.5, v_transposed=vt,
                                               out_dtype=out_dt, return_lse=True, causal_bottom_right=br, schedule=sched)
        torch.cuda.synchronize()
        outs[name] = (o.cpu().view(torch.uint8 if out_dt != torch.float16 else torch.int16).numpy(), lse.cpu().numpy())
    o_r, lse_r = outs["rolling"]
    for name in ("pipelined", "dense"):
        o_p, lse_p = outs[name]
        assert np.array_equal(o_r, o_p), f"{int((o_r != o_p).sum())} output elements differ between the rolling and the {name} loop"
        assert np.array_equal(lse_r.view(np.int32), lse_p.view(np.int32)), f"log-sum-exp differs between the rolling and the {name} loop"


@pytest.mark.parametrize("sched", [fa.FA8_SCHEDULE_ROLLING, fa.FA8_SCHEDULE_PIPELINED, fa.FA8_SCHEDULE_DENSE],
                         ids=["rolling", "pipelined", "dense"])
@pytest.mark.parametrize("causal", [False, True], ids=["full", "causal"])
def test_each_loop_against_the_oracle(sched, causal):
    B, H, N, d = 1, 2, 320, 128  # 5 whole blocks: the dense hint holds for the full-attention case
    q, k, v = _inputs(7, B, H, H, N, N, d, torch.float8_e4m3fn)
    scale = 0.11
    o = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale, schedule=sched)[0]
    torch.cuda.synchronize()
    u8 = [t.view(torch.uint8).numpy() for t in (q, k, v)]
    assert_parity(o.float().cpu().numpy(), *u8, scale, causal=causal, kv_block=fa.query(fa.FA8_QUERY_KV_BLOCK),
                  label=f"schedule {sched} causal {causal}")


def test_non_positive_scale_and_other_head_dims_ignore_the_hint():
    # the pipelined loop exists for head dims 64 / 128 and scale > 0; elsewhere the hint must be ignored, not rejected
    for d, scale in ((96, 0.1), (128, -0.1), (64, 0.0), (256, 0.06)):
        q, k, v = _inputs(3, 1, 2, 2, 200, 200, d, torch.float8_e4m3fn)
        a = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, scale, schedule=fa.FA8_SCHEDULE_PIPELINED)[0]
        b = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, scale, schedule=fa.FA8_SCHEDULE_ROLLING)[0]
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    with pytest.raises(RuntimeError):
        fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, 0.1, schedule=7)


def test_library_choice_by_launch_size():
    """fa8_fwd_schedule on the GPU box: full attention over whole KV blocks takes the dense loop; of the others, small launches
    take the pipelined loop and launches that fill the chip the rolling one."""
    import ctypes

    def plan(B, H, N, d, causal):
        q = torch.empty((B, H, N, d), dtype=torch.float8_e4m3fn, device=DEV)
        o = torch.empty((B, H, N, d), dtype=torch.float16, device=DEV)
        return fa.lib().fa8_fwd_schedule(ctypes.byref(fa.make_params(q, q, q, o, causal, d ** -0.5)))

    assert plan(1, 16, 1024, 128, True) == fa.FA8_SCHEDULE_PIPELINED      # 128 workgroups
    assert plan(4, 16, 1024, 64, False) == fa.FA8_SCHEDULE_DENSE          # cfg2
    assert plan(4, 16, 1000, 64, False) == fa.FA8_SCHEDULE_PIPELINED      # 512 workgroups with a ragged last block
    assert plan(4, 32, 2048, 64, True) == fa.FA8_SCHEDULE_PIPELINED       # 2048 short causal workgroups: little work per CU
    assert plan(2, 32, 4096, 128, False) == fa.FA8_SCHEDULE_DENSE         # the headline shape
    assert plan(2, 32, 4097, 128, False) == fa.FA8_SCHEDULE_ROLLING       # ... with a ragged last block
    assert plan(1, 32, 8192, 128, True) == fa.FA8_SCHEDULE_ROLLING        # cfg4
    assert plan(1, 16, 1024, 96, True) == fa.FA8_SCHEDULE_ROLLING         # no pipelined loop for this head dim
