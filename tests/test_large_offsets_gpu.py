"""Tensors of more than 2^31 elements (64-bit batch/head offsets) and a sequence length one past a multiple of every tile
size (N = 4097), checked on sampled heads and rows against the oracle in the device's arithmetic.

The reference forms one 32-bit head offset for q, k, v and o (reference csrc/flash_attention.cu:364) and has no tail
predication (:140, :152-154): both cases are beyond what it can run.
"""
import math

import numpy as np
import pytest
import torch

import cutlass_flash_atten_fp8_amd as fa
from oracle.parity_gate import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def u8(t):
    return t.view(torch.uint8).cpu().numpy()


@pytest.mark.parametrize("causal", [False, True])
def test_more_than_2_pow_31_elements_per_tensor(causal):
    B, H, N, d = 2, 2112, 4096, 128  # 2.21e9 elements per tensor: the second batch starts past 2^30, its last heads past 2^31
    need = B * H * N * d * (3 + 2) + (1 << 30)
    free, _ = torch.cuda.mem_get_info()
    if free < need:
        pytest.skip(f"needs {need >> 30} GiB of free device memory, {free >> 30} GiB available")
    assert B * H * N * d > 2 ** 31
    gen = torch.Generator(device=DEV).manual_seed(31)
    q, k, v = (torch.randn((B, H, N, d), device=DEV, generator=gen, dtype=torch.float16).to(torch.float8_e4m3fn) for _ in range(3))
    print(f"[large] bytes per tensor {q.numel()} causal={causal}", flush=True)
    scale = 1 / math.sqrt(d)
    o = fa.flash_attention_v2_cutlass(q, k, v, causal, scale)[0]
    torch.cuda.synchronize()
    rows = np.array([0, 1, 127, 128, 2047, 2048, 4000, 4095], dtype=np.int32)
    for b, h in ((0, 0), (0, H - 1), (1, 0), (1, 1000), (1, H - 2), (1, H - 1)):  # (1, H-1) ends at the last byte of each tensor
        sl = (slice(b, b + 1), slice(h, h + 1))
        got = o[sl].float().cpu().numpy()[:, :, rows]
        assert_parity(got, u8(q[sl]), u8(k[sl]), u8(v[sl]), scale, causal=causal, rows=rows, label=f"large b={b} h={h}",
                      reference_form=False)
    del q, k, v, o
    torch.cuda.empty_cache()


@pytest.mark.parametrize("causal", [False, True])
def test_sequence_length_4097(causal):
    """N = 4097 at d = 128: 32 full q blocks and one query row in the 33rd, 64 full kv blocks and one key in the 65th."""
    B, H, N, d = 1, 64, 4097, 128
    g = torch.Generator().manual_seed(4097)
    q, k, v = (torch.randn((B, H, N, d), generator=g).to(torch.float8_e4m3fn) for _ in range(3))
    scale = 1 / math.sqrt(d)
    o = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale)[0].float().cpu().numpy()
    rows = np.array(sorted({0, 1, 63, 64, 127, 128, 2048, 4031, 4032, 4094, 4095, 4096} | set(range(5, 4097, 67))), dtype=np.int32)
    assert_parity(o[:, :, rows], u8(q), u8(k), u8(v), scale, causal=causal, rows=rows, label=f"N=4097 causal={causal}")
