"""Build and install: libfa8.so (hipcc, gfx950), the PyTorch binding and the top-level module `attention_cutlass_fp8`
(the name the reference installs, reference setup.py:42-50).

    pip install .            or            python setup.py build_ext --inplace

The native build is the one of `python -m cutlass_flash_atten_fp8_amd.build` (plain hipcc for the kernels, plain g++ for
the host-only binding: no hipify, no CUDAExtension); the shared objects are shipped as package data.
"""
import os
import sys

from setuptools import Command, setup
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def native_build(force=False):
    from cutlass_flash_atten_fp8_amd import build as nb
    src = [os.path.join(nb.CSRC, f) for f in ("fa8_fwd_gfx950.hip", "attention_api.cpp")] + [os.path.join(nb.INCLUDE, "fa8_api.h")]
    newest = max(os.path.getmtime(f) for f in src)
    if force or not os.path.exists(nb.LIBFA8) or os.path.getmtime(nb.LIBFA8) < newest:
        nb.build_libfa8()
    if force or not os.path.exists(nb.EXT_PATH) or os.path.getmtime(nb.EXT_PATH) < newest:
        nb.build_binding()


class BuildNative(Command):
    description = "compile libfa8.so and the PyTorch binding in-tree"
    user_options = [("inplace", "i", "accepted for compatibility: the native build is always in-tree"),
                    ("force", "f", "rebuild even if the shared objects are newer than their sources")]
    boolean_options = ["inplace", "force"]

    def initialize_options(self):
        self.inplace = False
        self.force = False

    def finalize_options(self):
        pass

    def run(self):
        native_build(bool(self.force))


class BuildPyWithNative(build_py):
    def run(self):
        native_build()
        super().run()


setup(
    name="cutlass_flash_atten_fp8_amd",
    version="0.3.0",
    description="FP8 flash-attention forward for AMD MI355X (gfx950) behind the attention_cutlass_fp8 operator",
    packages=["cutlass_flash_atten_fp8_amd"],
    py_modules=["attention_cutlass_fp8"],
    package_data={"cutlass_flash_atten_fp8_amd": ["*.so", "csrc/fa8_fwd_gfx950.hip", "csrc/attention_api.cpp"]},
    cmdclass={"build_ext": BuildNative, "build_py": BuildPyWithNative},
    python_requires=">=3.9",
)
