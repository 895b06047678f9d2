"""Builds the native code of this package in-tree.

  libfa8.so                      hipcc --offload-arch=gfx950: kernels + C ABI (include/fa8_api.h)
  attention_cutlass_fp8.*.so     g++ host-only PyTorch binding that calls libfa8.so
  ../tests/cabi_host             g++: standalone C++ host of the C ABI (tests/test_cabi_host_gpu.py)

Run as `python -m cutlass_flash_atten_fp8_amd.build` or through __graft_entry__.build().
"""
import os
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
LIBFA8 = os.path.join(PKG_DIR, "libfa8.so")
EXT_NAME = "attention_cutlass_fp8"
EXT_PATH = os.path.join(PKG_DIR, EXT_NAME + sysconfig.get_config_var("EXT_SUFFIX"))

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # never let the compiler form packed fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError("command failed: " + " ".join(cmd))
    return r


def build_libfa8():
    cmd = [os.path.join(ROCM, "bin", "hipcc")] + HIPCC_FLAGS + ["-I", INCLUDE, "-o", LIBFA8,
                                                               os.path.join(CSRC, "fa8_fwd_gfx950.hip")]
    _run(cmd)
    return LIBFA8


def build_binding():
    import torch
    from torch.utils import cpp_extension
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = cpp_extension.include_paths()
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=" + EXT_NAME,
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I", INCLUDE, "-I", os.path.join(ROCM, "include"), "-I", sysconfig.get_paths()["include"]]
    for i in inc:
        cmd += ["-I", i]
    cmd += [os.path.join(CSRC, "attention_api.cpp"), "-o", EXT_PATH,
            "-L", PKG_DIR, "-l:libfa8.so", "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch", "-ltorch_python", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib]
    _run(cmd)
    return EXT_PATH


CABI_HOST_SRC = os.path.join(os.path.dirname(PKG_DIR), "tests", "cabi_host.cpp")
CABI_HOST = os.path.join(os.path.dirname(PKG_DIR), "tests", "cabi_host")


def build_cabi_host(force=False):
    """tests/cabi_host: the standalone C++ host of the C ABI used by tests/test_cabi_host_gpu.py (host code only)."""
    newest = max(os.path.getmtime(CABI_HOST_SRC), os.path.getmtime(os.path.join(INCLUDE, "fa8_api.h")))
    if force or not os.path.exists(CABI_HOST) or os.path.getmtime(CABI_HOST) < newest:
        _run(["g++", "-O2", "-std=c++17", "-D__HIP_PLATFORM_AMD__=1", "-I", INCLUDE, "-I", os.path.join(ROCM, "include"),
              CABI_HOST_SRC, "-o", CABI_HOST, "-L", PKG_DIR, "-l:libfa8.so", "-L", os.path.join(ROCM, "lib"), "-lamdhip64",
              "-Wl,-rpath," + PKG_DIR, "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return CABI_HOST


def build_all():
    build_libfa8()
    build_binding()
    # the C++ host of the C ABI is a test helper: failing to build it must not fail the product build
    if os.path.exists(CABI_HOST_SRC):
        try:
            build_cabi_host(force=True)
        except RuntimeError as e:
            sys.stderr.write("warning: tests/cabi_host was not built (%s)\n" % e)
    return LIBFA8, EXT_PATH


if __name__ == "__main__":
    for p in build_all():
        print("built", p)
