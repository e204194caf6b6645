"""Host-only checks (no GPU): the C-ABI library loads, exports every symbol
include/int4mm.h declares, and rejects bad arguments before touching the
device; the ``int4matmul`` extension exposes the reference's eleven entry points
(int4matmul.cpp:65-82) and fails loudly on CPU tensors."""
import ctypes as C
import os
import re

import pytest
import torch

import int4matmul_kernels_amd as pkg
from int4matmul_kernels_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "int4mm.h")).read()
    return sorted(set(re.findall(r"INT4MM_API\s+[\w\s\*]+?\b(int4mm_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    names = declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/int4mm.h but not exported"
    assert sorted(capi.EXPORTS) == names
    assert lib.int4mm_abi_version() == 1
    for code in range(0, 10):
        assert lib.int4mm_error_string(code)


def _call(fn, bits, shape, ptr=0x1000, mask=None, ws=0x1000, ws_bytes=1 << 30):
    sh = capi.Shape(*shape)
    vp = C.c_void_p
    return fn(bits, vp(ptr), vp(ptr), vp(ptr), vp(ptr), vp(ptr), vp(mask), C.byref(sh), vp(ws), ws_bytes, None)


def test_argument_validation_happens_on_the_host():
    lib = capi.lib()
    ok_vec = (1, 1, 128, 64, 16, 2, 64)          # B, M, K, S, R, G, g   (int4 dense)
    bad = {
        "bits": (lib.int4mm_matvec, 5, ok_vec, None, 1),
        "sparse with int3": (lib.int4mm_matvec, 3, (1, 1, 128, 64, 12, 2, 64), 0x1000, 2),
        "matvec with M=2": (lib.int4mm_matvec, 4, (1, 2, 128, 64, 16, 2, 64), None, 3),
        "K not multiple of 64": (lib.int4mm_matmul, 4, (1, 4, 96, 64, 12, 2, 64), None, 3),
        "S not multiple of 64": (lib.int4mm_matmul, 4, (1, 4, 128, 96, 16, 2, 64), None, 3),
        "packed rows mismatch": (lib.int4mm_matmul, 4, (1, 4, 128, 64, 15, 2, 64), None, 3),
        "sparse rows mismatch": (lib.int4mm_matmul, 4, (1, 4, 128, 64, 16, 2, 64), 0x1000, 3),
        "too few groups": (lib.int4mm_matmul, 4, (1, 4, 128, 64, 16, 1, 64), None, 3),
        "group size 32": (lib.int4mm_matmul, 4, (1, 4, 128, 64, 16, 4, 32), None, 4),
        "group size 0": (lib.int4mm_matmul, 4, (1, 4, 128, 64, 16, 4, 0), None, 4),
    }
    for what, (fn, bits, shape, mask, want) in bad.items():
        assert _call(fn, bits, shape, mask=mask) == want, what
    # null and misaligned pointers
    assert _call(lib.int4mm_matmul, 4, (1, 4, 128, 64, 16, 2, 64), ptr=None) == 5
    assert _call(lib.int4mm_matmul, 4, (1, 4, 128, 64, 16, 2, 64), ptr=0x1004) == 8
    # empty problems are accepted without a launch
    assert _call(lib.int4mm_matmul, 4, (0, 4, 128, 64, 16, 2, 64)) == 0
    assert _call(lib.int4mm_matvec, 4, (0, 1, 128, 64, 16, 2, 64)) == 0
    # helpers
    vp = C.c_void_p
    assert lib.int4mm_dense_pack(5, vp(16), vp(16), 64, 64, None) == 1
    assert lib.int4mm_dense_pack(4, vp(16), vp(16), 48, 64, None) == 3
    assert lib.int4mm_sparse_pack(vp(16), vp(16), vp(16), vp(16), 64, 48, None, None) == 3
    assert lib.int4mm_unpack(3, vp(16), None, vp(16), vp(16), 64, 64, None) == 2
    assert lib.int4mm_dequantize(4, vp(16), vp(16), vp(16), vp(16), None, 64, 64, 1, 32, None) == 4
    assert lib.int4mm_dequantize(4, None, vp(16), vp(16), vp(16), None, 64, 64, 1, 64, None) == 5
    assert lib.int4mm_workspace_bytes(20480) >= 20480 * 8
    # a NULL workspace names the array built into the library only together with a size of 0
    assert lib.int4mm_workspace_status(None, 4096, None) == 5
    assert lib.int4mm_workspace_init(None, 4096, None) == 5
    assert lib.int4mm_workspace_init(vp(4096), 16, None) == 6
    assert lib.int4mm_tune(99, 1) != 0 and lib.int4mm_tune(0, 0) == 0


def test_extension_surface_and_cpu_tensors_are_rejected():
    ext = pkg.load_extension()
    names = ["weight_matrix_packing", "quant_matmul"] + [
        f"quant_int{b}_linear_mult{suffix}" for b in (4, 3, 2) for suffix in ("", "_mtx", "_vec")]
    for n in names:
        assert callable(getattr(ext, n)), n
    import int4matmul                     # the reference's module name resolves to the same module
    assert int4matmul is ext
    outs = torch.zeros((1, 1, 64), dtype=torch.float16)
    matrix = torch.zeros((16, 64), dtype=torch.int32)
    x = torch.zeros((1, 1, 128), dtype=torch.float16)
    sz = torch.zeros((2, 64), dtype=torch.float16)
    with pytest.raises(ValueError):       # std::invalid_argument, as in the reference
        ext.quant_matmul(7, outs, matrix, x, sz, sz, 64, None)
    with pytest.raises(RuntimeError):     # no CPU path: tensors must be on the GPU
        ext.quant_matmul(4, outs, matrix, x, sz, sz, 64, None)
    with pytest.raises(RuntimeError):
        ext.weight_matrix_packing(matrix, matrix, torch.zeros((64, 128), dtype=torch.uint8),
                                  torch.zeros((64, 128), dtype=torch.uint8))
