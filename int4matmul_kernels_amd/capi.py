"""ctypes view of libint4mm_hip.so (include/int4mm.h) for torch tensors.

Every function takes tensors that already live on the GPU, passes raw device
pointers and the current HIP stream to the C ABI and raises ``Int4mmError`` on a
non-zero return code.  Nothing here computes anything.
"""
from __future__ import annotations

import ctypes as C
import os

_LIB = None
LIB_NAME = "libint4mm_hip.so"

EXPORTS = [
    "int4mm_error_string", "int4mm_last_hip_error", "int4mm_abi_version", "int4mm_tune",
    "int4mm_workspace_bytes", "int4mm_workspace_init", "int4mm_matmul_workspace_bytes", "int4mm_matvec", "int4mm_matmul",
    "int4mm_matvec_static", "int4mm_workspace_status", "int4mm_describe_launch",
    "int4mm_sparse_pack", "int4mm_dense_pack", "int4mm_unpack", "int4mm_dequantize",
]


class Int4mmError(RuntimeError):
    def __init__(self, code: int, what: str):
        self.code = code
        super().__init__(f"{what}: {lib().int4mm_error_string(code).decode()} (code {code})")


class Shape(C.Structure):
    _fields_ = [("batch", C.c_int64), ("seq_len", C.c_int64), ("in_size", C.c_int64),
                ("out_size", C.c_int64), ("matrix_rows", C.c_int64), ("n_groups", C.c_int64),
                ("group_size", C.c_int64)]


def lib_path() -> str:
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)


def lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(f"{path} is not built; run `python -m int4matmul_kernels_amd.build` "
                          "(there is no fallback implementation)")
    L = C.CDLL(path)
    vp, i64, sz = C.c_void_p, C.c_int64, C.c_size_t
    L.int4mm_error_string.restype = C.c_char_p
    L.int4mm_error_string.argtypes = [C.c_int]
    L.int4mm_last_hip_error.restype = C.c_int
    L.int4mm_abi_version.restype = C.c_int
    L.int4mm_tune.restype = C.c_int
    L.int4mm_tune.argtypes = [C.c_int, i64]
    L.int4mm_workspace_bytes.restype = sz
    L.int4mm_workspace_bytes.argtypes = [i64]
    L.int4mm_matmul_workspace_bytes.restype = sz
    L.int4mm_matmul_workspace_bytes.argtypes = [C.POINTER(Shape), C.c_int]
    L.int4mm_workspace_init.restype = C.c_int
    L.int4mm_workspace_init.argtypes = [vp, sz, vp]
    for name in ("int4mm_matvec", "int4mm_matmul"):
        f = getattr(L, name)
        f.restype = C.c_int
        f.argtypes = [C.c_int, vp, vp, vp, vp, vp, vp, C.POINTER(Shape), vp, sz, vp]
    L.int4mm_matvec_static.restype = C.c_int
    L.int4mm_matvec_static.argtypes = [C.c_int, vp, vp, vp, vp, vp, vp, C.POINTER(Shape), vp]
    L.int4mm_workspace_status.restype = C.c_int
    L.int4mm_workspace_status.argtypes = [vp, sz, vp]
    L.int4mm_describe_launch.restype = C.c_int
    L.int4mm_describe_launch.argtypes = [C.c_int, C.c_int, C.POINTER(Shape), C.c_int, sz, C.c_char_p, sz]
    L.int4mm_sparse_pack.restype = C.c_int
    L.int4mm_sparse_pack.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp]
    L.int4mm_dense_pack.restype = C.c_int
    L.int4mm_dense_pack.argtypes = [C.c_int, vp, vp, i64, i64, vp]
    L.int4mm_unpack.restype = C.c_int
    L.int4mm_unpack.argtypes = [C.c_int, vp, vp, vp, vp, i64, i64, vp]
    L.int4mm_dequantize.restype = C.c_int
    L.int4mm_dequantize.argtypes = [C.c_int, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp]
    _LIB = L
    return L


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc, what):
    if rc != 0:
        raise Int4mmError(rc, what)


def tune(key: int, value: int):
    _check(lib().int4mm_tune(key, value), "int4mm_tune")


def describe_launch(product, bits, batch, seq_len, in_size, out_size, group_size=128, sparse=False, workspace_bytes=None):
    """one line saying which kernel / tile shape / split ``matvec`` ("vec") or ``matmul`` ("mtx") would launch"""
    rows = in_size // 16 if sparse else in_size * bits // 32
    groups = 1 if group_size < 0 else -(-in_size // group_size)
    sh = Shape(batch, seq_len, in_size, out_size, rows, groups, group_size)
    if workspace_bytes is None:
        workspace_bytes = lib().int4mm_matmul_workspace_bytes(C.byref(sh), 1 if sparse else 0)
    buf = C.create_string_buffer(512)
    _check(lib().int4mm_describe_launch(0 if product == "vec" else 1, bits, C.byref(sh), 1 if sparse else 0,
                                        workspace_bytes, buf, 512), "int4mm_describe_launch")
    return buf.value.decode()


def workspace_status(workspace=None):
    """0 if healthy; raises Int4mmError(code 9) after a matvec hand-over timed out on it
    (``None``: the array built into the library that ``matvec_static`` works on)"""
    n = 0 if workspace is None else workspace.numel()
    _check(lib().int4mm_workspace_status(_ptr(workspace), n, _stream()), "int4mm_workspace_status")


def workspace_init(workspace=None):
    """zero-fill a workspace with a kernel on the current stream (``None``: the built-in array)"""
    n = 0 if workspace is None else workspace.numel()
    _check(lib().int4mm_workspace_init(_ptr(workspace), n, _stream()), "int4mm_workspace_init")


def new_workspace(out_size: int, device="cuda"):
    import torch
    n = lib().int4mm_workspace_bytes(out_size)
    return torch.zeros(n, dtype=torch.uint8, device=device)


def matmul_workspace_bytes(batch, seq_len, in_size, out_size, sparse=False) -> int:
    """bytes of workspace with which `matmul` may split K for this shape"""
    sh = Shape(batch, seq_len, in_size, out_size, 0, 0, 0)
    return lib().int4mm_matmul_workspace_bytes(C.byref(sh), 1 if sparse else 0)


def new_matmul_workspace(batch, seq_len, in_size, out_size, sparse=False, device="cuda"):
    import torch
    return torch.zeros(matmul_workspace_bytes(batch, seq_len, in_size, out_size, sparse), dtype=torch.uint8, device=device)


def _shape(outs, matrix, multiplier, scales, group_size):
    B, M, K = multiplier.shape
    G = scales.shape[0] if scales.dim() == 2 else 1
    return Shape(B, M, K, matrix.shape[1], matrix.shape[0], G, group_size)


def matvec(bits, outs, matrix, multiplier, scales, zeros, group_size, sparse_mask=None, workspace=None):
    sh = _shape(outs, matrix, multiplier, scales, group_size)
    nws = 0 if workspace is None else workspace.numel()
    _check(lib().int4mm_matvec(bits, _ptr(outs), _ptr(matrix), _ptr(multiplier), _ptr(scales),
                               _ptr(zeros), _ptr(sparse_mask), C.byref(sh), _ptr(workspace), nws,
                               _stream()), "int4mm_matvec")


def matvec_static(bits, outs, matrix, multiplier, scales, zeros, group_size, sparse_mask=None):
    """the matvec that allocates nothing: scratch is a device array built into the library"""
    sh = _shape(outs, matrix, multiplier, scales, group_size)
    _check(lib().int4mm_matvec_static(bits, _ptr(outs), _ptr(matrix), _ptr(multiplier), _ptr(scales),
                                      _ptr(zeros), _ptr(sparse_mask), C.byref(sh), _stream()), "int4mm_matvec_static")


def matmul(bits, outs, matrix, multiplier, scales, zeros, group_size, sparse_mask=None, workspace=None):
    sh = _shape(outs, matrix, multiplier, scales, group_size)
    nws = 0 if workspace is None else workspace.numel()
    _check(lib().int4mm_matmul(bits, _ptr(outs), _ptr(matrix), _ptr(multiplier), _ptr(scales),
                               _ptr(zeros), _ptr(sparse_mask), C.byref(sh), _ptr(workspace), nws,
                               _stream()), "int4mm_matmul")


def sparse_pack(wt_outs, msk_outs, wt_in, msk_in, bad_blocks=None):
    S, K = wt_in.shape
    _check(lib().int4mm_sparse_pack(_ptr(wt_outs), _ptr(msk_outs), _ptr(wt_in), _ptr(msk_in), S, K,
                                    _ptr(bad_blocks), _stream()), "int4mm_sparse_pack")


def dense_pack(bits, matrix_out, codes_in):
    K, S = codes_in.shape
    _check(lib().int4mm_dense_pack(bits, _ptr(matrix_out), _ptr(codes_in), K, S, _stream()),
           "int4mm_dense_pack")


def unpack(bits, codes_out, keep_out, matrix, sparse_mask=None):
    K, S = codes_out.shape
    _check(lib().int4mm_unpack(bits, _ptr(codes_out), _ptr(keep_out), _ptr(matrix), _ptr(sparse_mask),
                               K, S, _stream()), "int4mm_unpack")


def dequantize(bits, w_out, matrix, scales, zeros, group_size, sparse_mask=None):
    K, S = w_out.shape
    G = scales.shape[0] if scales.dim() == 2 else 1
    _check(lib().int4mm_dequantize(bits, _ptr(w_out), _ptr(matrix), _ptr(scales), _ptr(zeros),
                                   _ptr(sparse_mask), K, S, G, group_size, _stream()),
           "int4mm_dequantize")
