"""The import the reference's caller performs (reference test.py:3) works with nothing imported first, and setup.py
builds the native code and stages the package (module `attention_cutlass_fp8`, reference setup.py:45)."""
import glob
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _needs_toolchain():
    pkg = os.path.join(ROOT, "cutlass_flash_atten_fp8_amd")
    built = os.path.exists(os.path.join(pkg, "libfa8.so")) and glob.glob(os.path.join(pkg, "attention_cutlass_fp8.*.so"))
    hipcc = shutil.which("hipcc") or os.path.exists(os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc"))
    return not built and not hipcc


def run(args, cwd):
    return subprocess.run([sys.executable] + args, cwd=cwd, capture_output=True, text=True, timeout=600)


@pytest.mark.skipif(_needs_toolchain(), reason="the shared objects are not built and there is no hipcc to build them with")
def test_top_level_import_in_a_fresh_interpreter():
    code = ("import sys; assert not any(m.startswith('cutlass_flash_atten') for m in sys.modules); "
            "from attention_cutlass_fp8 import flash_attention_v2_cutlass as f; print(f.__doc__.splitlines()[0])")
    r = run(["-c", code], ROOT)
    assert r.returncode == 0, r.stderr
    assert "flash_attention_v2_cutlass" in r.stdout


@pytest.mark.skipif(_needs_toolchain(), reason="the shared objects are not built and there is no hipcc to build them with")
def test_setup_py_stages_the_package(tmp_path):
    r = run(["setup.py", "-q", "build", "--build-base", str(tmp_path / "b"), "--build-lib", str(tmp_path / "lib")], ROOT)
    assert r.returncode == 0, r.stdout + r.stderr
    staged = tmp_path / "lib"
    assert (staged / "attention_cutlass_fp8.py").exists()
    names = os.listdir(staged / "cutlass_flash_atten_fp8_amd")
    assert "libfa8.so" in names and any(n.startswith("attention_cutlass_fp8.") and n.endswith(".so") for n in names)
    # the staged copy imports from its own location
    code = "import attention_cutlass_fp8 as m, os; print(os.path.dirname(m.__file__))"
    r = run(["-c", code], str(staged))
    assert r.returncode == 0, r.stderr
    assert r.stdout.strip() == str(staged)
