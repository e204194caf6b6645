"""Shared helpers for the GPU parity tests: move an oracle problem to the GPU
and call the HIP path either through the C ABI (ctypes) or through the
``int4matmul`` extension module."""
import numpy as np
import torch

import int4matmul_kernels_amd as pkg
from int4matmul_kernels_amd import capi
from oracle import oracle as O

DEV = "cuda"


def t(a, dev=DEV):
    if a is None:
        return None
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def dev_problem(p):
    return dict(matrix=t(p["matrix"]), mask=t(p["sparse_mask"]), states=t(p["states"]),
                scales=t(p["scales"]), zeros=t(p["zeros"]))


def run_capi(p, d, kind, outs_init=None):
    B, M, S = p["B"], p["M"], p["S"]
    outs = torch.zeros((B, M, S), dtype=torch.float16, device=DEV) if outs_init is None \
        else t(outs_init).clone()
    # (the matvec's workspace plus room for split-K partial tiles where the shape wants them)
    ws = capi.new_matmul_workspace(B, M, p["K"], S, d["mask"] is not None)
    fn = capi.matvec if kind == "vec" else capi.matmul
    fn(p["bits"], outs, d["matrix"], d["states"], d["scales"], d["zeros"], p["group_size"],
       d["mask"], ws)
    torch.cuda.synchronize()
    return outs.cpu().numpy()


def run_ext(p, d, outs_init=None, fn_name="quant_matmul"):
    ext = pkg.load_extension()
    B, M, S = p["B"], p["M"], p["S"]
    outs = torch.zeros((B, M, S), dtype=torch.float16, device=DEV) if outs_init is None \
        else t(outs_init).clone()
    args = (outs, d["matrix"], d["states"], d["scales"], d["zeros"], p["group_size"], d["mask"])
    if fn_name == "quant_matmul":
        ext.quant_matmul(p["bits"], *args)
    else:
        getattr(ext, fn_name)(*args)
    torch.cuda.synchronize()
    return outs.cpu().numpy()


class OracleArray(np.ndarray):
    """an oracle's outputs, tagged with the bit width of the problem they belong to"""
    bits = None

    def __array_finalize__(self, obj):
        self.bits = getattr(obj, "bits", None)


def oracles(p):
    """(exact fp64 product on the fp16 weights, fp32 dequantise-then-matmul)"""
    w16 = O.dequantize_matrix(p["bits"], p["matrix"], p["scales"], p["zeros"], p["group_size"],
                              p["sparse_mask"])
    x = p["states"].reshape(-1, p["K"])
    exact = O.matmul_exact(x, w16).reshape(p["B"], p["M"], p["S"])
    linear_only = bool(np.all(p["scales"] >= 0))
    if linear_only:
        w32 = O.dequantize_matrix_fp32(p["bits"], p["matrix"], p["scales"], p["zeros"],
                                       p["group_size"], p["sparse_mask"])
        f32 = O.matmul_fp32(x, w32).reshape(p["B"], p["M"], p["S"])
    else:
        f32 = exact.astype(np.float32)
    f32 = f32.view(OracleArray)
    f32.bits = p["bits"]
    return exact, f32


# Tolerances (stated once, used by every product test):
#  * against fp32 dequantise-then-matmul: max relative error 1e-2, the bar of the
#    build's north star, denominators floored at the RMS of the true outputs;
#  * against the exact (float64) product on the fp16 weights the reference
#    multiplies: 2e-3 for the matmul, whose weights are those fp16 values bit for
#    bit (what is left is fp32 summation order and the fp16 output rounding,
#    4.9e-4 relative), with denominators floored at only 0.05 x RMS so that small
#    outputs are held to the same relative bar; 6e-3 (floor 1 x RMS) for the
#    matvec, which applies scale and zero in fp32
#    per group instead of rounding every weight to fp16 twice, so it differs
#    from that product by the weights' own rounding noise (and is closer to the
#    fp32 oracle than the reference is) -- and, because of that, the matvec class is also
#    held to 3e-3 of the fp32 oracle itself with the tight floor of 0.05 x RMS (linear
#    quantisation; what is left there is the fp16 output rounding and the fp32 summation of
#    x * (2^e + q), whose rounding is absolute: about 2^-24 of the magic offsets times the
#    scale), so that a kernel which corrupted small outputs could not pass on the wide floor.
#    int3 / int2 in the benchmark's scale range (up to 0.08, four times int4's, on codes of
#    0 .. 3 riding on offsets of up to 1024) get 1.2e-2 on the same floor (worst seen: 9.6e-3, int2 at K = 256);
#  * the reference's own gate: mean relative error <= 0.1 (kernel_test.py:344-348).
TOL_F32 = 1e-2
TOL_EXACT = 6e-3          # matvec
TOL_VEC_F32 = 3e-3        # matvec against the fp32 oracle, denominators max(|truth|, 0.05 x RMS): int4
TOL_VEC_F32_NARROW = 1.2e-2  # ... int3 / int2
TOL_EXACT_MTX = 2e-3      # matmul
FLOOR_EXACT_MTX = 0.05    # its denominators: max(|truth|, 0.05 x RMS)
TOL_MEAN = 0.1


def matmul_kind(p):
    """tolerance class of a matmul call: "mtx" when a kernel that dequantises its weights (tile
    kernels, the 17 .. 256 row kernel) serves the shape, "vec" when the 2 .. 96 row kernel does,
    which -- like the matvec -- applies scale and zero per group in fp32"""
    line = capi.describe_launch("mtx", p["bits"], p["B"], p["M"], p["K"], p["S"], p["group_size"], p["sparse_mask"] is not None)
    return "vec" if line.startswith("skinny_kernel") or p["B"] * p["M"] == 1 else "mtx"


def assert_product_close(got, exact, f32, prior=None, kind="vec", tight=None):
    """`tight`: also hold the result to the fp32 oracle with the tight floor -- for the kernels that apply scale
    and zero in fp32 per group (the matvec and the 2 .. 16 row kernel).  Default: every single-row product (the
    matvec kernel serves them all); tests of the few-row kernel ask for it."""
    bits = getattr(f32, "bits", None)
    if tight is None:
        tight = kind == "vec" and exact.size == exact.shape[-1]
    # (problems with exponent-mode groups have no fp32 oracle of their own: `oracles` hands back the exact product)
    stand_in = np.array_equal(f32, exact.astype(np.float32))
    if prior is not None:
        exact = exact + prior.astype(np.float64)
        f32 = f32 + prior.astype(np.float32)
    assert np.all(np.isfinite(got.astype(np.float32)))
    e1 = O.max_rel_error(exact, got, floor_frac=1.0 if kind == "vec" else FLOOR_EXACT_MTX)
    e2 = O.max_rel_error(f32, got)
    if tight and not stand_in:
        # (the fp32-per-group kernels follow the fp32 dequantise-then-matmul oracle closely, small outputs included)
        e4 = O.max_rel_error(f32, got, floor_frac=FLOOR_EXACT_MTX)
        assert e4 < (TOL_VEC_F32 if bits in (None, 4) else TOL_VEC_F32_NARROW), f"vs fp32 oracle, tight floor: {e4}"
    # the reference's metric (mean of |error| / |truth|) over the outputs that are not next to zero: a single
    # output whose true value is 1e-6 of the others' turns a rounding error into a ratio of thousands (or, at
    # exactly zero, into inf), and among 1e5 ... 1e7 outputs there are such
    nz = np.abs(f32) >= 1e-3 * np.max(np.abs(f32))
    e3 = O.mean_rel_error(f32[nz], got[nz])
    assert e1 < (TOL_EXACT if kind == "vec" else TOL_EXACT_MTX), f"vs exact product: {e1}"
    assert e2 < TOL_F32, f"vs fp32 oracle: {e2}"
    assert e3 < TOL_MEAN, f"mean relative error: {e3}"
    return e1, e2, e3
