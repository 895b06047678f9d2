"""The reference's CPU-runnable path, restated: naive attention in PyTorch on the fp8-cast inputs.

TEST INFRASTRUCTURE ONLY; bench.py times it as the `cpu_baseline`.  It is a port of `self_attention`
(reference test.py:25-33): S = Q K^T * scale, optional lower-triangular mask, fp32 softmax, P V --
with the two deviations the fp8 pipeline prescribes: the fp8 inputs are upcast to fp32 before the
matmuls (the reference upcasts to fp16 on the GPU), and the softmax numerator is re-quantised to e4m3
before P V while the denominator keeps the fp32 P (reference csrc/flash_attention.cu:524, :268-271).
Works one (batch, head) at a time so the N x N score matrix stays small.
"""
import torch


def naive_attention_cpu(q8, k8, v8, scale, causal=False, heads_limit=None):
    """q8, k8, v8: CPU tensors float8_e4m3fn [B,H,N,d].  Returns fp16 [B,H,N,d] (or the first
    `heads_limit` (batch*head) slices when given, for a bounded timing sample)."""
    B, H, N, d = q8.shape
    nk = k8.shape[2]
    qf = q8.reshape(B * H, N, d)
    kf = k8.reshape(B * H, nk, d)
    vf = v8.reshape(B * H, nk, d)
    n = B * H if heads_limit is None else min(B * H, heads_limit)
    out = torch.empty((n, N, d), dtype=torch.float16)
    mask = None
    if causal:
        mask = torch.ones((N, nk), dtype=torch.bool).tril_()
    for i in range(n):
        s = (qf[i].float() @ kf[i].float().T) * scale
        if mask is not None:
            s = s.masked_fill(~mask, float("-inf"))
        p = torch.exp(s - s.max(dim=-1, keepdim=True).values)
        l = p.sum(dim=-1, keepdim=True)
        p8 = p.to(torch.float8_e4m3fn).float()
        out[i] = ((p8 @ vf[i].float()) / l).half()
    return out if heads_limit is not None else out.reshape(B, H, N, d)
