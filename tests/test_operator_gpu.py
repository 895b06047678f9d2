"""GPU tests of the operator boundary: the compiled binding `attention_cutlass_fp8`, the ctypes mirror and the raw C ABI
must agree bit for bit; streams, determinism, guard bands, strided tensors, fp8 output, e5m2 inputs, error paths."""
import ctypes
import math

import numpy as np
import pytest
import torch

import cutlass_flash_atten_fp8_amd as fa
from oracle import fa8_oracle as fo
from oracle.parity_gate import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rand_fp8(shape, seed, dtype=torch.float8_e4m3fn, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def u8(t):
    return t.view(torch.uint8).cpu().numpy()


def abi_call(q, k, v, o, causal, scale, stream=None):
    p = fa.make_params(q, k, v, o, causal, scale)
    s = torch.cuda.current_stream() if stream is None else stream
    rc = fa.lib().fa8_fwd(ctypes.byref(p), ctypes.c_void_p(s.cuda_stream))
    assert rc == 0, fa.error_string(rc)
    return o


@pytest.mark.parametrize("causal", [False, True])
def test_binding_mirror_and_abi_agree_bitwise(causal):
    ext = fa.load_extension()
    q, k, v = (rand_fp8((2, 4, 300, 128), s).to(DEV) for s in (1, 2, 3))
    out = ext.flash_attention_v2_cutlass(q, k, v, causal, 0.09)
    assert isinstance(out, list) and len(out) == 1
    o1 = out[0]
    assert o1.dtype == torch.float16 and o1.shape == q.shape and o1.is_contiguous()
    o2 = fa.flash_attention_v2_cutlass(q, k, v, causal, 0.09)[0]
    o3 = abi_call(q, k, v, torch.empty_like(o1), causal, 0.09)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(o1, o3)
    # keyword form of the five reference arguments
    o4 = ext.flash_attention_v2_cutlass(q=q, k=k, v=v, is_causal=causal, softmax_scale=0.09)[0]
    assert torch.equal(o1, o4)


def test_runs_on_the_current_stream_without_device_sync():
    ext = fa.load_extension()
    q, k, v = (rand_fp8((1, 8, 1024, 128), s).to(DEV) for s in (4, 5, 6))
    ref = ext.flash_attention_v2_cutlass(q, k, v, False, 0.09)[0]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        o = ext.flash_attention_v2_cutlass(q, k, v, False, 0.09)[0]
        done = torch.cuda.Event()
        done.record(side)
    done.synchronize()
    assert torch.equal(o, ref)


def test_deterministic_run_to_run():
    q, k, v = (rand_fp8((2, 8, 2000, 128), s).to(DEV) for s in (7, 8, 9))
    outs = [fa.flash_attention_v2_cutlass(q, k, v, True, 0.09)[0] for _ in range(3)]
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


@pytest.mark.parametrize("n,d", [(1, 64), (100, 64), (129, 128), (1000, 128), (70, 32), (130, 96), (200, 160), (333, 224), (65, 256)])
def test_guard_bands_and_poisoned_padding(n, d):
    """O is written only inside [B,H,N,d]; K/V bytes past row N-1 (NaN codes here) never reach the result."""
    B, H, pad = 2, 2, 64
    qs, ks, vs = (rand_fp8((B, H, n, d), s) for s in (10, 11, 12))

    def padded(t):  # rows n..n+pad of every head are fp8 NaN (0x7F)
        buf = torch.full((B, H, n + pad, d), 0x7F, dtype=torch.uint8)
        buf[:, :, :n] = t.view(torch.uint8)
        return buf.to(DEV).view(torch.float8_e4m3fn)[:, :, :n]

    qp, kp, vp = padded(qs), padded(ks), padded(vs)
    obuf = torch.full((B, H, n + pad, d), 777.0, dtype=torch.float16, device=DEV)
    abi_call(qp, kp, vp, obuf[:, :, :n], False, 0.1)
    o_plain = abi_call(qs.to(DEV), ks.to(DEV), vs.to(DEV), torch.empty((B, H, n, d), dtype=torch.float16, device=DEV), False, 0.1)
    torch.cuda.synchronize()
    assert torch.equal(obuf[:, :, :n], o_plain)
    assert (obuf[:, :, n:] == 777.0).all()
    assert torch.isfinite(o_plain).all()


def test_strided_batch_and_head_layout():
    """[B,N,H,d] storage viewed as [B,H,N,d]: arbitrary batch/head/row strides, last dim contiguous."""
    B, H, n, d = 2, 3, 200, 128
    qs, ks, vs = (rand_fp8((B, n, H, d), s).to(DEV) for s in (13, 14, 15))
    q, k, v = (t.permute(0, 2, 1, 3) for t in (qs, ks, vs))
    o = torch.empty((B, n, H, d), dtype=torch.float16, device=DEV).permute(0, 2, 1, 3)
    abi_call(q, k, v, o, True, 0.09)
    ref = abi_call(q.contiguous(), k.contiguous(), v.contiguous(), torch.empty((B, H, n, d), dtype=torch.float16, device=DEV), True, 0.09)
    torch.cuda.synchronize()
    assert torch.equal(o.contiguous(), ref)


def test_causal_rows_do_not_see_future_keys_bitwise():
    q, k, v = (rand_fp8((1, 4, 700, 128), s) for s in (16, 17, 18))
    a = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, 0.09)[0]
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 400:] = rand_fp8((1, 4, 300, 128), 19, scale=3.0)
    v2[:, :, 400:] = rand_fp8((1, 4, 300, 128), 20, scale=3.0)
    b = fa.flash_attention_v2_cutlass(q.to(DEV), k2.to(DEV), v2.to(DEV), True, 0.09)[0]
    torch.cuda.synchronize()
    assert torch.equal(a[:, :, :400], b[:, :, :400])
    assert not torch.equal(a[:, :, 400:], b[:, :, 400:])


def test_closed_form_answers_on_the_gpu():
    d, n = 128, 300
    q, k, v = (rand_fp8((1, 2, n, d), s) for s in (21, 22, 23))
    # causal row 0 is exactly V[0]
    o = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, 0.09)[0].cpu()
    assert torch.equal(o[:, :, 0].float(), v[:, :, 0].float())
    # scale 0: every visible weight is exactly 1 -> O = (prefix) mean of V
    o0 = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), False, 0.0)[0].float().cpu()
    assert torch.allclose(o0, v.float().mean(dim=2, keepdim=True).expand_as(o0), atol=1e-3, rtol=0)
    oc = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), True, 0.0)[0].float().cpu()
    prefix = torch.cumsum(v.float(), dim=2) / torch.arange(1, n + 1).view(1, 1, n, 1)
    assert torch.allclose(oc, prefix, atol=2e-3, rtol=0)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2], ids=["e4m3", "e5m2"])
@pytest.mark.parametrize("d", [32, 64, 96, 128, 160, 192, 224, 256])
def test_fp8_output_matches_oracle(causal, d, dtype):
    """out_dtype = the fp8 type of the inputs: what the reference itself stores (reference csrc/flash_attention.cu:557,
    convert_float32_to_fp8<Element>, into empty_like(q), :655-656)."""
    e5m2 = dtype == torch.float8_e5m2
    q, k, v = (rand_fp8((2, 2, 260, d), s, dtype=dtype) for s in (24, 25, 26))
    scale = 1 / math.sqrt(d)
    o8 = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale, out_dtype=dtype)[0]
    o16 = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale)[0]
    assert o8.dtype == dtype
    # same fp32 result rounded once to fp8 and once to fp16: the fp8 output must be within half an fp8 step of the fp16 one
    a, b = o8.float().cpu().numpy(), o16.float().cpu().numpy()
    half_step = np.maximum(np.abs(b) * 2.0 ** (-3 if e5m2 else -4), 2.0 ** (-17 if e5m2 else -10))
    assert np.all(np.abs(a - b) <= half_step * 1.001)
    # against the oracle in the device's arithmetic with the same output type: the codes are identical except where the fp32
    # value sits within an ulp of a rounding boundary (the device's exp2 and the CPU's differ by an ulp), and then adjacent
    ref = fo.forward(u8(q), u8(k), u8(v), scale, causal=causal, exp2_form=True, matmul_model=fo.MATMUL_GFX950,
                     in_dtype=fo.E5M2 if e5m2 else fo.E4M3, out_dtype=fo.OUT_E5M2 if e5m2 else fo.OUT_E4M3)
    refv = torch.from_numpy(ref).view(dtype).float().numpy()
    differ = a != refv
    print(f"fp8 out d={d} causal={causal} {'e5m2' if e5m2 else 'e4m3'}: {differ.mean() * 100:.3f} % of codes differ", flush=True)
    assert differ.mean() < 0.005
    assert np.all(np.abs(a - refv)[differ] <= 2 * half_step[differ] * 1.001)
    # a mixed pair (fp8 output of the other format) is rejected
    other = torch.float8_e4m3fn if e5m2 else torch.float8_e5m2
    with pytest.raises(RuntimeError):
        fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale, out_dtype=other)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("d", [32, 64, 96, 128, 160, 192, 224, 256])
def test_e5m2_inputs_match_oracle(causal, d):
    q, k, v = (rand_fp8((2, 2, 333, d), s, dtype=torch.float8_e5m2) for s in (27, 28, 29))
    scale = 1 / math.sqrt(d)
    o = fa.flash_attention_v2_cutlass(q.to(DEV), k.to(DEV), v.to(DEV), causal, scale)[0].float().cpu().numpy()
    assert_parity(o, u8(q), u8(k), u8(v), scale, causal=causal, in_dtype=fo.E5M2, label=f"e5m2 d={d} causal={causal}")


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("n,d", [(64, 64), (208, 64), (256, 128), (1008, 128), (80, 32), (528, 32), (64, 256), (400, 256), (144, 96), (320, 160),
                                 (192, 192), (272, 224)])
def test_transposed_v_is_the_reference_calling_convention(n, d, causal):
    """v_transposed=True takes v as [B,H,d,N], what the reference requires of its caller (reference test.py:71);
    the result is bit-identical to the [B,H,N,d] call."""
    ext = fa.load_extension()
    q, k, v = (rand_fp8((2, 3, n, d), s).to(DEV) for s in (40, 41, 42))
    o = ext.flash_attention_v2_cutlass(q, k, v, causal, 0.1)[0]
    vt = v.transpose(2, 3).contiguous()
    ot = ext.flash_attention_v2_cutlass(q, k, vt, causal, 0.1, v_transposed=True)[0]
    torch.cuda.synchronize()
    assert torch.equal(o, ot)
    assert_parity(ot.float().cpu().numpy(), u8(q), u8(k), u8(vt), 0.1, causal=causal, v_transposed=True,
                  label=f"transposed v n={n} d={d} causal={causal}")


def test_error_paths_raise_and_launch_nothing():
    ext = fa.load_extension()
    q = rand_fp8((1, 2, 128, 80), 30).to(DEV)
    with pytest.raises(RuntimeError, match="head_dim"):
        ext.flash_attention_v2_cutlass(q, q, q, False, 0.1)
    q = rand_fp8((1, 2, 128, 128), 31).to(DEV)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.flash_attention_v2_cutlass(q.transpose(1, 2), q, q, False, 0.1)
    with pytest.raises(RuntimeError, match="same dtype"):
        ext.flash_attention_v2_cutlass(q, q.view(torch.uint8).view(torch.float8_e5m2), q, False, 0.1)
    with pytest.raises(RuntimeError, match="float8"):
        ext.flash_attention_v2_cutlass(q.half(), q.half(), q.half(), False, 0.1)
    with pytest.raises(RuntimeError, match="float8"):
        ext.flash_attention_v2_cutlass(*(t.view(torch.uint8).view(torch.float8_e4m3fnuz) for t in (q, q, q)), False, 0.1)
    k3 = rand_fp8((1, 3, 128, 128), 32).to(DEV)
    with pytest.raises(RuntimeError, match="multiple"):  # 2 q heads over 3 k/v heads
        ext.flash_attention_v2_cutlass(q, k3, k3, True, 0.1)
    with pytest.raises(RuntimeError, match="finite"):
        ext.flash_attention_v2_cutlass(q, q, q, False, float("nan"))
    q100 = rand_fp8((1, 2, 100, 128), 33).to(DEV)
    with pytest.raises(RuntimeError, match="aligned"):  # the [B,H,d,N] layout is read in 16-byte chunks along N
        ext.flash_attention_v2_cutlass(q100, q100, q100.transpose(2, 3).contiguous(), False, 0.1, v_transposed=True)
    torch.cuda.synchronize()
    # seqlen_q != seqlen_k is fine without the causal mask
    k_short = rand_fp8((1, 2, 64, 128), 34).to(DEV)
    o = ext.flash_attention_v2_cutlass(q, k_short, k_short, False, 0.1)[0]
    ref = fo.forward(u8(q), u8(k_short), u8(k_short), 0.1, exp2_form=True).astype(np.float32)
    assert np.abs(o.float().cpu().numpy() - ref).mean() <= 2e-3


@pytest.mark.parametrize("schedule,causal", [(fa.FA8_SCHEDULE_ROLLING, True), (fa.FA8_SCHEDULE_PIPELINED, True),
                                             (fa.FA8_SCHEDULE_DENSE, False)], ids=["rolling", "pipelined", "dense"])
def test_capturable_in_a_hip_graph(schedule, causal):
    """The launcher allocates nothing and never synchronises, so the operator can be recorded into a HIP graph
    (here through torch.cuda.graph, whose allocator provides the output inside the capture) and replayed; all main loops."""
    ext = fa.load_extension()
    q, k, v = (rand_fp8((2, 4, 384, 128), s).to(DEV) for s in (50, 51, 52))
    eager = ext.flash_attention_v2_cutlass(q, k, v, causal, 0.09, schedule=schedule)[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture, as torch asks
        ext.flash_attention_v2_cutlass(q, k, v, causal, 0.09, schedule=schedule)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ext.flash_attention_v2_cutlass(q, k, v, causal, 0.09, schedule=schedule)[0]
    for i in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"
        # eager work and new inputs between replays: the graph reads q/k/v in place
        q.copy_(rand_fp8((2, 4, 384, 128), 60 + i).to(DEV))
        eager = ext.flash_attention_v2_cutlass(q, k, v, causal, 0.09, schedule=schedule)[0].clone()


@pytest.mark.parametrize("nk,causal,schedule", [(99968, False, fa.FA8_SCHEDULE_AUTO), (100000, False, fa.FA8_SCHEDULE_PIPELINED),
                                                (100000, True, fa.FA8_SCHEDULE_ROLLING), (100000, True, fa.FA8_SCHEDULE_PIPELINED)])
def test_long_kv_with_rows_far_apart(nk, causal, schedule):
    """100 000 keys whose rows lie 20 480 bytes apart: the kernel's 32-bit byte offsets into k and v run up to 2.05e9, just
    under the 2^31 the library accepts.  The gaps between the rows hold NaN codes, so a misplaced read shows.  Bit for bit the
    result of the same call on contiguous copies, and a few rows against the oracle."""
    d, nq, stride = 128, 200, 20480
    q, k, v = (rand_fp8((1, 1, n, d), s).to(DEV) for n, s in ((nq, 31), (nk, 32), (nk, 33)))
    wide = []
    for t in (k, v):
        big = torch.full((nk, stride), 0x7F, dtype=torch.uint8, device=DEV)
        big[:, :d] = t.view(torch.uint8)[0, 0]
        wide.append(big[:, :d].view(torch.float8_e4m3fn)[None, None])
    kw, vw = wide
    assert kw.stride(2) == stride and kw.shape == k.shape
    scale = 1.0 / math.sqrt(d)
    outs = []
    for kk, vv in ((kw, vw), (k, v)):
        o = torch.empty((1, 1, nq, d), dtype=torch.float16, device=DEV)
        p = fa.make_params(q, kk, vv, o, causal, scale, causal_bottom_right=True, schedule=schedule)
        rc = fa.lib().fa8_fwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, fa.error_string(rc)
        outs.append(o)
    torch.cuda.synchronize()
    assert torch.isfinite(outs[0]).all()
    assert torch.equal(outs[0], outs[1])
    rows = np.array([0, 1, 63, 64, 127, 128, nq - 1], dtype=np.int32)
    want = fo.forward(u8(q), u8(k), u8(v), scale, causal=causal, rows=rows, exp2_form=True, causal_bottom_right=True,
                      matmul_model=fo.MATMUL_GFX950).astype(np.float32)
    got = outs[0].float().cpu().numpy()[:, :, rows]
    assert np.abs(got - want).max() <= 2e-2 and np.abs(got - want).mean() <= 2e-3  # the parity bar
