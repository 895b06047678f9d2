"""A standalone C++ program (tests/cabi_host.cpp: no Python, no PyTorch) drives libfa8.so through the C ABI of
include/fa8_api.h on the golden inputs; its output bytes must equal what the same call gives through ctypes."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import cutlass_flash_atten_fp8_amd as fa
from cutlass_flash_atten_fp8_amd import build as native_build

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("causal", [0, 1])
def test_cpp_host_matches_ctypes_bitwise(tmp_path, causal):
    import torch
    host = native_build.build_cabi_host()  # compiled beforehand by __graft_entry__.build(); built here only if missing
    G = np.load(os.path.join(HERE, "golden", "cfg1_golden.npz"))
    B, H, N, d = G["q"].shape
    for name in ("q", "k", "v"):
        G[name].tofile(tmp_path / f"{name}.bin")
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.dirname(fa.LIBFA8_PATH) + ":" + os.environ.get("LD_LIBRARY_PATH", ""))
    r = subprocess.run([host, str(B), str(H), str(N), str(d), str(causal), repr(float(G["scale"])), str(tmp_path / "q.bin"),
                        str(tmp_path / "k.bin"), str(tmp_path / "v.bin"), str(tmp_path / "o.bin")], capture_output=True,
                       text=True, timeout=120, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "o.bin", dtype=np.uint16).reshape(B, H, N, d)
    dev = torch.device("cuda:0")
    q, k, v = (torch.from_numpy(G[n]).to(dev).view(torch.float8_e4m3fn) for n in ("q", "k", "v"))
    o = torch.empty(q.shape, dtype=torch.float16, device=dev)
    p = fa.make_params(q, k, v, o, bool(causal), float(G["scale"]))
    rc = fa.lib().fa8_fwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, fa.error_string(rc)
    torch.cuda.synchronize()
    assert np.array_equal(got, o.view(torch.int16).cpu().numpy().view(np.uint16))
