"""``import int4matmul`` -- the reference's module name (setup.py:5-8, kernel_test.py:6).

The compiled extension lives inside the ``int4matmul_kernels_amd`` package, beside the
C-ABI library it links to.  This file, next to the package on ``sys.path``, makes the
reference's own import line work unchanged: it loads the compiled module and puts it
in ``sys.modules`` under this name, so ``int4matmul.quant_matmul`` and the ten other
entry points (int4matmul.cpp:65-82) are the compiled functions themselves.  torch is
imported first, as every torch extension needs.  No fallback: a missing build raises
ImportError.
"""
import sys

import torch  # noqa: F401  (the extension links to libtorch)

sys.modules.pop(__name__, None)          # (so that the loader does not mistake this file for the module)
from int4matmul_kernels_amd import load_extension as _load_extension  # noqa: E402

sys.modules[__name__] = _load_extension()
