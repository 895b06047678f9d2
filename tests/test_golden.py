"""Golden vectors (tests/golden/cfg1_golden.npz, written by tests/golden/make_golden.py with this repository's
oracle): the oracle must keep reproducing them bit for bit, and on a GPU the kernel must meet the tolerance on them."""
import ctypes
import os

import numpy as np
import pytest

from oracle import fa8_oracle as fo
from oracle import np_restatement as nr
from oracle.parity_gate import assert_parity

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cfg1_golden.npz"))


def test_oracle_reproduces_golden_bits():
    o = fo.forward(G["q"], G["k"], G["v"], float(G["scale"]), kv_block=int(G["kv_block"]))
    oc = fo.forward(G["q"], G["k"], G["v"], float(G["scale"]), causal=True, kv_block=int(G["kv_block"]))
    assert np.array_equal(o.view(np.uint16), G["o_fp16_bits"])
    assert np.array_equal(oc.view(np.uint16), G["o_causal_fp16_bits"])


def test_numpy_restatement_close_to_golden():
    o = nr.forward(G["q"], G["k"], G["v"], float(G["scale"]), kv_block=int(G["kv_block"]))
    err = np.abs(o.astype(np.float32) - G["o_fp16_bits"].view(np.float16).astype(np.float32))
    assert np.median(err) == 0 and err.mean() < 1e-4


def test_golden_is_within_the_pipeline_error_of_exact_attention():
    err = np.abs(G["o_fp16_bits"].view(np.float16).astype(np.float32) - G["o_exact_f32"])
    assert err.max() < 3e-2 and err.mean() < 4e-3


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [False, True])
def test_kernel_on_golden(causal):
    import torch
    import cutlass_flash_atten_fp8_amd as fa
    assert fa.query(fa.FA8_QUERY_KV_BLOCK) == int(G["kv_block"])
    dev = torch.device("cuda:0")
    q, k, v = (torch.from_numpy(G[n]).to(dev).view(torch.float8_e4m3fn) for n in ("q", "k", "v"))
    o = torch.empty(q.shape, dtype=torch.float16, device=dev)
    p = fa.make_params(q, k, v, o, causal, float(G["scale"]))
    rc = fa.lib().fa8_fwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, fa.error_string(rc)
    torch.cuda.synchronize()
    got = o.float().cpu().numpy()
    assert_parity(got, G["q"], G["k"], G["v"], float(G["scale"]), causal=causal, kv_block=int(G["kv_block"]), label="golden cfg1")
    # and against the committed bits themselves (the oracle in the reference's arithmetic form): strict as well
    want = G["o_causal_fp16_bits" if causal else "o_fp16_bits"].view(np.float16).astype(np.float32)
    err = np.abs(got - want)
    assert err.max() <= 2e-2 and err.mean() <= 2e-3, (float(err.max()), float(err.mean()))
