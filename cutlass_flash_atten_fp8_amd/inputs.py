"""Seeded synthetic inputs for the benchmark configurations (all generated on the CPU, then cast to fp8).

The reference draws N(0, 0.5) fp16, clamps to +-0.1 and casts to e4m3 (reference test.py:13-23), which makes the
softmax nearly uniform; the configurations here keep full-range logits instead so that the softmax numerics,
masking and P quantisation are exercised.
"""
import math

import torch

# name -> (B, H, N, d, causal, distribution)
CONFIGS = {
    "cfg1": dict(B=1, H=2, N=128, d=64, causal=False, dist="normal", seed=1001),
    "cfg2": dict(B=4, H=16, N=1024, d=64, causal=False, dist="normal", seed=1002),
    "cfg3": dict(B=2, H=32, N=4096, d=128, causal=False, dist="normal", seed=1003),
    "cfg4": dict(B=1, H=32, N=8192, d=128, causal=True, dist="normal_half", seed=1004),
    "cfg5": dict(B=1, H=8, N=16000, d=128, causal=True, dist="student_t", seed=1005),
}


def softmax_scale(cfg):
    return 1.0 / math.sqrt(cfg["d"])


def flops(cfg):
    """4*B*H*N^2*d, halved for causal."""
    f = 4.0 * cfg["B"] * cfg["H"] * cfg["N"] * cfg["N"] * cfg["d"]
    return f / 2 if cfg["causal"] else f


def algorithmic_bytes(cfg, out_bytes=2):
    """q + k + v read once (1 byte each) and o written once."""
    return cfg["B"] * cfg["H"] * cfg["N"] * cfg["d"] * (3 + out_bytes)


def make_qkv(cfg, dtype=torch.float8_e4m3fn):
    """Returns CPU fp8 tensors q, k, v of shape [B,H,N,d]."""
    g = torch.Generator(device="cpu").manual_seed(cfg["seed"])
    shape = (cfg["B"], cfg["H"], cfg["N"], cfg["d"])
    dist = cfg["dist"]
    if dist in ("normal", "normal_half"):
        s = 0.5 if dist == "normal_half" else 1.0
        q, k, v = (torch.randn(shape, generator=g, dtype=torch.float32) * s for _ in range(3))
    elif dist == "student_t":
        # Student-t(3) = N(0,1) / sqrt(chi2(3)/3): heavy-tailed logits, clipped to the e4m3 range; v ~ U(-1, 1)
        def student():
            z = torch.randn(shape, generator=g, dtype=torch.float32)
            chi = sum(torch.randn(shape, generator=g, dtype=torch.float32) ** 2 for _ in range(3))
            return (z / torch.sqrt(chi / 3.0)).clamp_(-448.0, 448.0)
        q, k = student(), student()
        v = torch.rand(shape, generator=g, dtype=torch.float32) * 2.0 - 1.0
    else:
        raise ValueError(dist)
    return q.to(dtype), k.to(dtype), v.to(dtype)
