"""Top-level name of the reference's extension module (reference setup.py:45, imported at reference test.py:3):

    from attention_cutlass_fp8 import flash_attention_v2_cutlass

This file only locates the compiled binding that cutlass_flash_atten_fp8_amd builds in-tree
(cutlass_flash_atten_fp8_amd/attention_cutlass_fp8.*.so, source csrc/attention_api.cpp) and re-exports it, so that the
import above works with nothing imported first.  There is no Python or CPU implementation behind it: a missing binding
or a missing libfa8.so raises ImportError.
"""
import importlib.util as _util
import os as _os
import sysconfig as _sysconfig

_pkg = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "cutlass_flash_atten_fp8_amd")
_path = _os.path.join(_pkg, "attention_cutlass_fp8" + _sysconfig.get_config_var("EXT_SUFFIX"))
if not _os.path.exists(_path) or not _os.path.exists(_os.path.join(_pkg, "libfa8.so")):
    raise ImportError(f"{_path} or libfa8.so beside it is missing: build them with `python -m cutlass_flash_atten_fp8_amd.build` "
                      "or `pip install .` (there is no fallback implementation)")
import torch as _torch  # noqa: E402,F401  (the binding links against libtorch)

_spec = _util.spec_from_file_location("attention_cutlass_fp8", _path)
_ext = _util.module_from_spec(_spec)
_spec.loader.exec_module(_ext)
flash_attention_v2_cutlass = _ext.flash_attention_v2_cutlass
kv_block = _ext.kv_block
__doc__ = _ext.__doc__ or __doc__
