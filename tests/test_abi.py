"""C-ABI boundary, CPU only: libfa8.so loads, exports every function include/fa8_api.h declares, and the host-side
argument validation returns the documented codes without touching a GPU.  No compute entry point is called with
arguments that would pass validation."""
import ctypes
import os
import re

import pytest
import torch

import cutlass_flash_atten_fp8_amd as fa

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = []
    for fn in os.listdir(os.path.join(ROOT, "include")):
        if fn.endswith(".h"):
            text = open(os.path.join(ROOT, "include", fn)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names += re.findall(r"^\s*(?:const\s+)?(?:int|char\s*\*|void)\s*\*?\s*(fa8_\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_header_declares_the_expected_entry_points():
    assert declared_functions() == sorted(fa.FA8_EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(fa.LIBFA8_PATH)
    for name in declared_functions():
        assert getattr(lib, name) is not None


def test_query_values():
    assert fa.query(fa.FA8_QUERY_VERSION) >= 1
    assert fa.query(fa.FA8_QUERY_KV_BLOCK) in (64, 128)
    assert fa.query(fa.FA8_QUERY_PARAMS_SIZE) == ctypes.sizeof(fa.Fa8FwdParams)  # the ctypes mirror has the C layout
    assert fa.query(fa.FA8_QUERY_VERSION) >= 2
    assert fa.query(fa.FA8_QUERY_Q_BLOCK) % 32 == 0
    assert fa.query(fa.FA8_QUERY_KV_ASCENDING) == 1
    assert fa.query(fa.FA8_QUERY_THREADS) % 64 == 0
    assert fa.query(12345) == -1
    assert fa.error_string(0) == "ok"
    assert "head_dim" in fa.error_string(-3)
    assert fa.error_string(-999)


@pytest.mark.skipif(__import__("shutil").which("gcc") is None, reason="no C compiler")
def test_header_is_plain_c_and_the_ctypes_mirror_has_its_layout(tmp_path):
    """include/fa8_api.h compiles as strict C99 on its own, and every field of Fa8FwdParams sits where the ctypes mirror
    puts it (offset and size, taken from a C program built against the header), as do the numeric codes."""
    import subprocess
    fields = [name for name, _ in fa.Fa8FwdParams._fields_]
    codes = ["FA8_DTYPE_E4M3", "FA8_DTYPE_E5M2", "FA8_OUT_FP16", "FA8_OUT_E4M3", "FA8_OUT_E5M2", "FA8_V_ROWS", "FA8_V_TRANSPOSED",
             "FA8_CAUSAL_TOP_LEFT", "FA8_CAUSAL_BOTTOM_RIGHT", "FA8_SCHEDULE_AUTO", "FA8_SCHEDULE_ROLLING",
             "FA8_SCHEDULE_PIPELINED", "FA8_SCHEDULE_DENSE", "FA8_QUERY_VERSION", "FA8_QUERY_KV_BLOCK", "FA8_QUERY_Q_BLOCK",
             "FA8_QUERY_KV_ASCENDING", "FA8_QUERY_THREADS", "FA8_QUERY_PARAMS_SIZE"]
    src = tmp_path / "layout.c"
    lines = ['#include "fa8_api.h"', "#include <stddef.h>", "#include <stdio.h>", "int main(void) {",
             '  printf("sizeof %zu\\n", sizeof(Fa8FwdParams));']
    for f in fields:
        lines.append(f'  printf("{f} %zu %zu\\n", offsetof(Fa8FwdParams, {f}), sizeof(((Fa8FwdParams*)0)->{f}));')
    for c in codes:
        lines.append(f'  printf("{c} %d\\n", (int){c});')
    lines += ["  return 0;", "}"]
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), str(src),
                    "-o", str(exe)], check=True, capture_output=True)
    out = dict((ln.split()[0], [int(x) for x in ln.split()[1:]]) for ln in
               subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    assert out["sizeof"] == [ctypes.sizeof(fa.Fa8FwdParams)]
    for f in fields:
        d = getattr(fa.Fa8FwdParams, f)
        assert out[f] == [d.offset, d.size], f
    assert len(out) == 1 + len(fields) + len(codes)
    for c in codes:
        assert out[c] == [getattr(fa, c)], c


def cpu_tensors(n=64, d=64, dtype=torch.float8_e4m3fn, b=1, h=2):
    q = torch.zeros((b, h, n, d), dtype=torch.float32).to(dtype)
    return q, q.clone(), q.clone(), torch.zeros((b, h, n, d), dtype=torch.float16)


def validate(p):
    return fa.lib().fa8_fwd_validate(ctypes.byref(p))


def test_validate_accepts_a_plain_problem():
    q, k, v, o = cpu_tensors()
    assert validate(fa.make_params(q, k, v, o, False, 0.125)) == 0
    assert validate(fa.make_params(q, k, v, o, True, 0.125)) == 0
    o8 = torch.zeros(o.shape, dtype=torch.float32).to(torch.float8_e4m3fn)
    assert validate(fa.make_params(q, k, v, o8, False, 0.125)) == 0


def test_validate_rejects_bad_arguments():
    q, k, v, o = cpu_tensors()
    assert fa.lib().fa8_fwd_validate(None) == -1
    p = fa.make_params(q, k, v, o, False, 0.125); p.q = None
    assert validate(p) == -1
    p = fa.make_params(q, k, v, o, False, 0.125); p.seqlen_k = 0
    assert validate(p) == -2
    p = fa.make_params(q, k, v, o, True, 0.125); p.seqlen_k = 32
    assert validate(p) == 0  # causal with seqlen_q != seqlen_k: top-left aligned by default
    p.causal_align = fa.FA8_CAUSAL_BOTTOM_RIGHT
    assert validate(p) == 0
    p.causal_align = 2
    assert validate(p) == -6
    p = fa.make_params(q, k, v, o, False, 0.125); p.heads_k = 3  # 2 q heads
    assert validate(p) == -2
    p.heads_k = -1
    assert validate(p) == -2
    for hk in (0, 1, 2):
        p.heads_k = hk
        assert validate(p) == 0
    lse = torch.zeros((1, 2, 64), dtype=torch.float32)
    p = fa.make_params(q, k, v, o, False, 0.125, lse=lse)
    assert validate(p) == 0
    p.lse_head_stride = 63
    assert validate(p) == -4
    p = fa.make_params(q, k, v, o, False, 0.125, lse=lse); p.lse = p.lse + 2
    assert validate(p) == -5
    for d in (16, 48, 80, 288, 512):
        q2, k2, v2, o2 = cpu_tensors(d=d)
        assert validate(fa.make_params(q2, k2, v2, o2, False, 0.125)) == -3
    for d in (32, 64, 96, 128, 160, 192, 224, 256):  # the reference's head-dim buckets (static_switch.h:50-77)
        q2, k2, v2, o2 = cpu_tensors(d=d)
        assert validate(fa.make_params(q2, k2, v2, o2, False, 0.125)) == 0
    p = fa.make_params(q, k, v, o, False, 0.125); p.k_row_stride = 32
    assert validate(p) == -4
    p = fa.make_params(q, k, v, o, False, 0.125); p.k_row_stride = 72
    assert validate(p) == -5
    p = fa.make_params(q, k, v, o, False, 0.125); p.q = p.q + 4
    assert validate(p) == -5
    p = fa.make_params(q, k, v, o, False, 0.125); p.in_dtype = 7
    assert validate(p) == -6
    p = fa.make_params(q, k, v, o, False, 0.125); p.out_dtype = 9
    assert validate(p) == -6
    vt = torch.zeros((1, 2, 64, 72), dtype=torch.float32).to(torch.float8_e4m3fn)[..., :64]  # [B,H,d,N], row stride 72
    p = fa.make_params(q, k, vt, o, False, 0.125, v_transposed=True)
    assert validate(p) == -5
    vt = torch.zeros((1, 2, 64, 64), dtype=torch.float32).to(torch.float8_e4m3fn)
    assert validate(fa.make_params(q, k, vt, o, False, 0.125, v_transposed=True)) == 0
    for bad in (float("nan"), float("inf")):
        assert validate(fa.make_params(q, k, v, o, False, bad)) == -8


def test_fa8_fwd_rejects_before_any_gpu_work():
    # invalid arguments must come back as negative codes even on a machine without a GPU
    q, k, v, o = cpu_tensors(d=80)
    p = fa.make_params(q, k, v, o, False, 0.125)
    assert fa.lib().fa8_fwd(ctypes.byref(p), None) == -3


def test_python_operator_mirrors_reference_errors():
    q, k, v, _ = cpu_tensors()
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fa.flash_attention_v2_cutlass(q, k, v, False, 0.125)
    with pytest.raises(TypeError):
        fa.flash_attention_v2_cutlass(q, k, v)  # all five arguments are required, as in the reference binding


def test_compiled_binding_mirrors_reference_errors():
    ext = fa.load_extension()
    import attention_cutlass_fp8
    assert attention_cutlass_fp8 is ext
    q, k, v, _ = cpu_tensors()
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ext.flash_attention_v2_cutlass(q, k, v, False, 0.125)
    with pytest.raises(TypeError):
        ext.flash_attention_v2_cutlass(q, k, v)
    assert ext.kv_block() == fa.query(fa.FA8_QUERY_KV_BLOCK)


def test_schedule_query_follows_explicit_hints_without_a_gpu():
    """fa8_fwd_schedule: an explicit hint is answered without touching the GPU; it holds only where the loop it names exists."""
    sched = fa.lib().fa8_fwd_schedule
    for d, scale, hint, want in ((128, 0.1, fa.FA8_SCHEDULE_PIPELINED, fa.FA8_SCHEDULE_PIPELINED),
                                 (64, 0.1, fa.FA8_SCHEDULE_PIPELINED, fa.FA8_SCHEDULE_PIPELINED),
                                 (128, 0.1, fa.FA8_SCHEDULE_ROLLING, fa.FA8_SCHEDULE_ROLLING),
                                 (96, 0.1, fa.FA8_SCHEDULE_PIPELINED, fa.FA8_SCHEDULE_ROLLING),
                                 (256, 0.1, fa.FA8_SCHEDULE_AUTO, fa.FA8_SCHEDULE_ROLLING),
                                 (128, -0.1, fa.FA8_SCHEDULE_PIPELINED, fa.FA8_SCHEDULE_ROLLING),
                                 (64, 0.0, fa.FA8_SCHEDULE_AUTO, fa.FA8_SCHEDULE_ROLLING)):
        q, k, v, o = cpu_tensors(d=d)
        p = fa.make_params(q, k, v, o, True, scale, schedule=hint)
        assert sched(ctypes.byref(p)) == want, (d, scale, hint)
    # the dense loop: full attention, seqlen_k a multiple of the KV block, head dim 64 / 128, positive scale; chosen without a hint
    for d, n, scale, hint, want in ((128, 128, 0.1, fa.FA8_SCHEDULE_AUTO, fa.FA8_SCHEDULE_DENSE),
                                    (64, 64, 0.1, fa.FA8_SCHEDULE_DENSE, fa.FA8_SCHEDULE_DENSE),
                                    (128, 128, 0.1, fa.FA8_SCHEDULE_ROLLING, fa.FA8_SCHEDULE_ROLLING),
                                    (128, 128, 0.1, fa.FA8_SCHEDULE_PIPELINED, fa.FA8_SCHEDULE_PIPELINED),
                                    (96, 128, 0.1, fa.FA8_SCHEDULE_DENSE, fa.FA8_SCHEDULE_ROLLING),
                                    (128, 128, 0.0, fa.FA8_SCHEDULE_DENSE, fa.FA8_SCHEDULE_ROLLING)):
        q, k, v, o = cpu_tensors(n=n, d=d)
        p = fa.make_params(q, k, v, o, False, scale, schedule=hint)
        assert sched(ctypes.byref(p)) == want, (d, n, scale, hint)
    q, k, v, o = cpu_tensors()
    p = fa.make_params(q, k, v, o, False, 0.1, schedule=9)
    assert sched(ctypes.byref(p)) == -6 and validate(p) == -6  # FA8_ERR_DTYPE: unknown schedule code
    assert sched(None) == -1
    p = fa.make_params(q, k, v, o, False, 0.1)
    p.reserved0 = 1
    assert validate(p) == -7  # FA8_ERR_UNSUPPORTED: a field of a later version of the parameter block is set
