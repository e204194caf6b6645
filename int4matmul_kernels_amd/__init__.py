"""MI355X-native int{4,3,2} x fp16 matvec / matmul.

Two binaries live beside this file (built by ``int4matmul_kernels_amd.build``):

* ``libint4mm_hip.so`` -- the C-ABI library declared in ``include/int4mm.h``;
  ``capi`` wraps it with ctypes for torch tensors.
* ``int4matmul.*.so``  -- the drop-in Python extension with the reference's entry
  points; ``load_extension()`` imports it and registers it as ``int4matmul``.

There is no CPU or pure-PyTorch fallback: if a binary is missing the loaders
raise ImportError.
"""
from __future__ import annotations

import importlib.util
import os
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
__all__ = ["load_extension", "capi", "PKG_DIR"]


def load_extension():
    """Import the compiled ``int4matmul`` module (and make ``import int4matmul``
    resolve to it).  torch must be imported first: the module links to it."""
    if "int4matmul" in sys.modules:
        return sys.modules["int4matmul"]
    import sysconfig

    import torch  # noqa: F401  (loads libtorch / the HIP runtime the module links to)

    path = os.path.join(PKG_DIR, "int4matmul" + sysconfig.get_config_var("EXT_SUFFIX"))
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is not built; run `python -m int4matmul_kernels_amd.build` "
            "(there is no fallback implementation)")
    spec = importlib.util.spec_from_file_location("int4matmul", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    sys.modules["int4matmul"] = mod
    return mod


from . import capi  # noqa: E402
