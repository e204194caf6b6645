"""CPU oracle for the quantized int{4,3,2} x fp16 matvec / matmul path.

TEST INFRASTRUCTURE ONLY.  This module restates, in numpy, what the reference
CUDA kernels compute.  It is imported by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` as
the checker; the product (the HIP library and the ``int4matmul`` extension)
never imports it and has no CPU fallback.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  How each function is pinned independently of its own
formula is listed beside it ("pinned by").  ``dequant_exponent`` and the
negative-scale switch have no test or fixture in the reference
(kernel_test.py:58 leaves them as a TODO): they are pinned by tables of fp16
bit patterns typed by hand from the reference's text (every code of every bit
width, the added zero, the negated scale, the single rounding, -0.0 and NaN
scales) in tests/test_oracle.py.

Dimension names: K = reduction dim (unpacked weight rows), S = output columns,
R = packed rows, g = group size.
"""
from __future__ import annotations

import numpy as np

SUPPORTED_BITS = (4, 3, 2)
ONE_GROUP = 0x0FFFFFFF  # matmul_kernel.cu:379-381, matvec_kernel.cu:307-309


# --------------------------------------------------------------------------
# F1/F2: dense power-of-two packing  (packer kernel_test.py:60-80;
# decoders matmul.cuh:246-268 and matvec_kernel.cu:17-51)
# pinned by: brute-force single-code columns, pack/unpack round trip, and the
# C restatement of the decoder's shift loop in oracle/oracle_c.c.
# --------------------------------------------------------------------------
def pack_dense_pow2(bits: int, codes: np.ndarray) -> np.ndarray:
    """codes uint8/int [K, S] -> int32 [K*bits/32, S]; code k of a word at bits
    ``bits*(k mod (32/bits))``, LSB first."""
    assert bits in (4, 2)
    per = 32 // bits
    K, S = codes.shape
    assert K % per == 0
    c = codes.astype(np.uint32).reshape(K // per, per, S)
    sh = (np.arange(per, dtype=np.uint32) * bits)[None, :, None]
    words = np.bitwise_or.reduce(c << sh, axis=1).astype(np.uint32)
    return words.view(np.int32)


def unpack_dense_pow2(bits: int, matrix: np.ndarray) -> np.ndarray:
    """int32 [R, S] -> uint8 codes [R*32/bits, S]."""
    assert bits in (4, 2)
    per = 32 // bits
    w = np.ascontiguousarray(matrix).view(np.uint32)
    R, S = w.shape
    sh = (np.arange(per, dtype=np.uint32) * bits)[None, :, None]
    codes = (w[:, None, :] >> sh) & np.uint32((1 << bits) - 1)
    return codes.reshape(R * per, S).astype(np.uint8)


# --------------------------------------------------------------------------
# F3: dense int3 packing: every 32 codes of a column are a 96-bit LSB-first
# bitstream over 3 consecutive packed rows (packer kernel_test.py:82-123;
# decoders matmul.cuh:270-309 and matvec_kernel.cu:53-127).
# pinned by: one-hot codes at each of the 32 positions against the word/bit
# positions the two reference decoders read; round trip; C restatement.
# --------------------------------------------------------------------------
def pack_dense_int3(codes: np.ndarray) -> np.ndarray:
    K, S = codes.shape
    assert K % 32 == 0
    c = codes.astype(np.uint64).reshape(K // 32, 32, S)
    out = np.zeros((K // 32, 3, S), dtype=np.uint32)
    lo = np.zeros((K // 32, S), dtype=np.uint64)   # stream bits 0..63
    hi = np.zeros((K // 32, S), dtype=np.uint64)   # stream bits 64..95
    for j in range(32):
        pos = 3 * j
        v = c[:, j, :] & np.uint64(7)
        if pos + 3 <= 64:
            lo |= v << np.uint64(pos)
        elif pos >= 64:
            hi |= v << np.uint64(pos - 64)
        else:  # straddles bit 64 (j == 21: bits 63,64,65)
            lo |= (v << np.uint64(pos)) & np.uint64(0xFFFFFFFFFFFFFFFF)
            hi |= v >> np.uint64(64 - pos)
    out[:, 0, :] = (lo & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    out[:, 1, :] = (lo >> np.uint64(32)).astype(np.uint32)
    out[:, 2, :] = (hi & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    return out.reshape(K // 32 * 3, S).view(np.int32)


def unpack_dense_int3(matrix: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(matrix).view(np.uint32)
    R, S = w.shape
    assert R % 3 == 0
    w = w.reshape(R // 3, 3, S).astype(np.uint64)
    lo = w[:, 0, :] | (w[:, 1, :] << np.uint64(32))
    hi = w[:, 2, :]
    codes = np.zeros((R // 3, 32, S), dtype=np.uint8)
    for j in range(32):
        pos = 3 * j
        if pos + 3 <= 64:
            v = lo >> np.uint64(pos)
        elif pos >= 64:
            v = hi >> np.uint64(pos - 64)
        else:
            v = (lo >> np.uint64(pos)) | (hi << np.uint64(64 - pos))
        codes[:, j, :] = (v & np.uint64(7)).astype(np.uint8)
    return codes.reshape(R // 3 * 32, S)


def pack_dense(bits: int, codes: np.ndarray) -> np.ndarray:
    if bits == 3:
        return pack_dense_int3(codes)
    return pack_dense_pow2(bits, codes)


def unpack_dense(bits: int, matrix: np.ndarray) -> np.ndarray:
    if bits == 3:
        return unpack_dense_int3(matrix)
    return unpack_dense_pow2(bits, matrix)


# --------------------------------------------------------------------------
# F4: 16:32 sparse int4 (packer utils_kernel.cu:19-64, shapes :84-95;
# decoders matmul.cuh:334-405 (dropped rows decode to 0.0, :398) and
# matvec_kernel.cu:135-169).
# pinned by: popcount invariant, decode(pack(w, m)) == w*m, the fixed
# "keep lower/upper 16" masks reducing to F1 on half the rows, C restatement
# of the packer's ballot/popc/shift-add loop.
# --------------------------------------------------------------------------
def sparse_pack(codes_sk: np.ndarray, keep_sk: np.ndarray):
    """Inputs in the packer's orientation: uint8 [S, K] codes and keep mask
    (>0 = keep, utils_kernel.cu:34).  Returns (weights int32 [K/16, S],
    mask int32 [K/32, S])."""
    S, K = codes_sk.shape
    assert K % 32 == 0
    keep = (keep_sk > 0).reshape(S, K // 32, 32)
    if not np.all(keep.sum(axis=2) == 16):          # utils_kernel.cu:41
        raise ValueError("every 32-row block must keep exactly 16 rows")
    code = (codes_sk.astype(np.uint64) & np.uint64(0xF)).reshape(S, K // 32, 32)
    bitpos = np.arange(32, dtype=np.uint64)[None, None, :]
    mask = np.bitwise_or.reduce(keep.astype(np.uint64) << bitpos, axis=2)
    rank = np.cumsum(keep, axis=2) - keep            # popc(mask & ((1<<t)-1))
    v = np.where(keep, code << (np.uint64(4) * rank.astype(np.uint64)), np.uint64(0))
    v = np.bitwise_or.reduce(v, axis=2)              # 64-bit compacted codes
    wt = np.empty((K // 32, 2, S), dtype=np.uint32)
    wt[:, 0, :] = (v & np.uint64(0xFFFFFFFF)).astype(np.uint32).T
    wt[:, 1, :] = (v >> np.uint64(32)).astype(np.uint32).T
    msk = mask.astype(np.uint32).T
    return (wt.reshape(K // 16, S).view(np.int32),
            np.ascontiguousarray(msk).view(np.int32))


def sparse_unpack(matrix: np.ndarray, mask: np.ndarray):
    """(weights int32 [K/16,S], mask int32 [K/32,S]) -> (codes uint8 [K,S],
    keep bool [K,S]).  Rank based like both reference decoders; dropped rows
    get code 0 and keep False."""
    w = np.ascontiguousarray(matrix).view(np.uint32)
    m = np.ascontiguousarray(mask).view(np.uint32)
    nb, S = m.shape
    assert w.shape == (2 * nb, S)
    w = w.reshape(nb, 2, S).astype(np.uint64)
    v = w[:, 0, :] | (w[:, 1, :] << np.uint64(32))
    t = np.arange(32, dtype=np.uint32)[None, :, None]
    keep = ((m[:, None, :] >> t) & np.uint32(1)).astype(bool)      # [nb,32,S]
    rank = np.cumsum(keep, axis=1) - keep
    sh = np.minimum(rank, 15).astype(np.uint64) * np.uint64(4)
    codes = ((v[:, None, :] >> sh) & np.uint64(0xF)).astype(np.uint8)
    codes = np.where(keep, codes, np.uint8(0))
    return codes.reshape(nb * 32, S), keep.reshape(nb * 32, S)


# --------------------------------------------------------------------------
# Dequantisation (matmul.cuh:115-136) and the per (group, column) switch
# (matmul.cuh:414-428, matvec_kernel.cu:178-190).
# pinned by (linear): IEEE-754: numpy float16 subtract and multiply are each
# correctly rounded, as __hsub/__hmul are; checked exhaustively against an
# independent float64-then-round evaluation in tests.  Exponent mode: closed
# form in float64 rounded once (a power of two times s is exact); checked against
# hand-typed fp16 bit patterns for every code of every bit width in tests.
# --------------------------------------------------------------------------
def dequant_linear(codes, scale, zero):
    """fp16( fp16( fp16(q) - z ) * s )  -- matmul.cuh:117-121."""
    q = np.asarray(codes).astype(np.float16)
    return ((q - np.asarray(zero, dtype=np.float16)).astype(np.float16)
            * np.asarray(scale, dtype=np.float16)).astype(np.float16)


def dequant_exponent(bits: int, codes, pos_scale, zero):
    """fp16_fma( +-2^(v & (2^(bits-1)-1)), s', z ), sign = bit bits-1 of the code;
    s' is the negated (hence positive) stored scale -- matmul.cuh:127-136."""
    v = np.asarray(codes).astype(np.int64)
    mag = np.left_shift(1, v & ((1 << (bits - 1)) - 1)).astype(np.float64)
    iv = np.where(v & (1 << (bits - 1)), -mag, mag)
    r = iv * np.asarray(pos_scale, dtype=np.float16).astype(np.float64) \
        + np.asarray(zero, dtype=np.float16).astype(np.float64)
    return r.astype(np.float16)    # one rounding: the product is exact in f64


def dequant_dynamic(bits: int, codes, scale, zero):
    """scale >= 0 -> linear, else exponent mode with -scale (matmul.cuh:420).
    ``-0.0 >= 0`` is true; NaN scale takes the exponent branch."""
    scale = np.asarray(scale, dtype=np.float16)
    zero = np.asarray(zero, dtype=np.float16)
    lin = dequant_linear(codes, scale, zero)
    with np.errstate(invalid="ignore"):
        ex = dequant_exponent(bits, codes, -scale, zero)
        return np.where(scale >= np.float16(0), lin, ex).astype(np.float16)


def group_index(K: int, group_size: int) -> np.ndarray:
    g = ONE_GROUP if group_size < 0 else group_size
    return (np.arange(K) // g).astype(np.int64)


def _expand_groups(param: np.ndarray, K: int, group_size: int) -> np.ndarray:
    p = np.asarray(param)
    if p.ndim == 1:                      # single-group [S] form, kernel_test.py:177-179
        p = p[None, :]
    return p[group_index(K, group_size)]    # [K, S]


def dequantize_matrix(bits, matrix, scales, zeros, group_size, sparse_mask=None):
    """Packed weights -> fp16 [K, S] exactly as the kernels' unpack step builds
    the fp16 tile (matmul.cuh:246-405): bit-exact target for the HIP dequantize
    helper.  Dropped rows of the sparse format are exactly 0.0."""
    if sparse_mask is not None:
        if bits != 4:
            raise ValueError("16:32 sparsity exists for int4 only")   # matmul.cuh:184-190
        codes, keep = sparse_unpack(matrix, sparse_mask)
    else:
        codes, keep = unpack_dense(bits, matrix), None
    K = codes.shape[0]
    s = _expand_groups(scales, K, group_size)
    z = _expand_groups(zeros, K, group_size)
    w = dequant_dynamic(bits, codes, s, z)
    if keep is not None:
        w = np.where(keep, w, np.float16(0))
    return w


def dequantize_matrix_fp32(bits, matrix, scales, zeros, group_size, sparse_mask=None):
    """fp32 dequantisation, (q - z) * s with every operand widened first: the
    "hiW" matrix of kernel_test.py:141,152 and the north-star fp32 oracle.
    Linear mode only (the harness never builds exponent-mode data)."""
    if sparse_mask is not None:
        codes, keep = sparse_unpack(matrix, sparse_mask)
    else:
        codes, keep = unpack_dense(bits, matrix), None
    K = codes.shape[0]
    s = _expand_groups(scales, K, group_size).astype(np.float32)
    z = _expand_groups(zeros, K, group_size).astype(np.float32)
    w = (codes.astype(np.float32) - z) * s
    if keep is not None:
        w = np.where(keep, w, np.float32(0))
    return w.astype(np.float32)


# --------------------------------------------------------------------------
# Products.  Kernel semantics: matmul overwrites outs with
# fp16(sum_k fp32(x) * fp32(w_fp16)) (matmul_kernel.cu:219-333); matvec
# accumulates onto the prior contents, outs = fp16(fp32(outs) + x.W)
# (matvec_kernel.cu:351,381-382).  Summation order is not defined by the
# reference (atomics / WMMA), so products are compared within tolerance.
# --------------------------------------------------------------------------
def matmul_fp32(x: np.ndarray, w32: np.ndarray) -> np.ndarray:
    """north-star oracle: fp32 states @ fp32 dequantised weights
    (kernel_test.py:251-252)."""
    return x.astype(np.float32) @ w32


def matmul_exact(x: np.ndarray, w16: np.ndarray) -> np.ndarray:
    """Tighter oracle: fp16-dequantised weights (what the kernels multiply),
    float64 accumulation; returns float64."""
    return x.astype(np.float64) @ w16.astype(np.float64)


def matvec_expected(outs_old: np.ndarray, y: np.ndarray) -> np.ndarray:
    """Accumulate-into-outs quirk of the matvec launcher."""
    return (outs_old.astype(np.float32) + y.astype(np.float32)).astype(np.float16)


# --------------------------------------------------------------------------
# Error metrics
# --------------------------------------------------------------------------
def mean_rel_error(truth: np.ndarray, cand: np.ndarray) -> float:
    """nanmean(|cand - truth| / |truth|)  -- kernel_test.py:261-262; the
    reference's pass rule is <= 0.1 (kernel_test.py:344-348)."""
    with np.errstate(divide="ignore", invalid="ignore"):
        r = np.abs((cand.astype(np.float64) - truth.astype(np.float64)) / truth.astype(np.float64))
    return float(np.nanmean(r))


def max_rel_error(truth: np.ndarray, cand: np.ndarray, floor_frac: float = 1.0) -> float:
    """max |cand - truth| / max(|truth|, floor_frac * rms(truth)).

    Element-wise relative error is ill-conditioned where the true output is
    near zero (an fp16 result cannot be within 1 % of a value that is itself
    smaller than the rounding error of its summands), so denominators are
    floored at ``floor_frac`` times the RMS of the true outputs."""
    t = truth.astype(np.float64)
    c = cand.astype(np.float64)
    rms = float(np.sqrt(np.mean(t * t))) if t.size else 0.0
    den = np.maximum(np.abs(t), max(floor_frac * rms, np.finfo(np.float64).tiny))
    return float(np.max(np.abs(c - t) / den)) if t.size else 0.0


# --------------------------------------------------------------------------
# Seeded synthetic workloads of the benchmark shapes.  Generated with numpy on the
# CPU so that every machine sees identical bits.
# --------------------------------------------------------------------------
def make_problem(K, S, M=1, bits=4, group_size=128, sparse=False, seed=0, B=1,
                 scale_range=(0.001, 0.02), zero_range=(0.0, 15.0), zero_const=None):
    """Returns a dict with states fp16 [B,M,K], codes uint8 [K,S], matrix int32,
    sparse_mask int32|None, keep bool [K,S]|None, scales/zeros fp16 [G,S]."""
    rng = np.random.default_rng(seed)
    states = rng.standard_normal((B, M, K), dtype=np.float32).astype(np.float16)
    codes = rng.integers(0, 1 << bits, size=(K, S), dtype=np.uint8)
    G = 1 if group_size < 0 else -(-K // group_size)
    scales = rng.uniform(scale_range[0], scale_range[1], size=(G, S)).astype(np.float16)
    if zero_const is not None:
        zeros = np.full((G, S), zero_const, dtype=np.float16)
    else:
        zeros = rng.uniform(zero_range[0], zero_range[1], size=(G, S)).astype(np.float16)
    keep = None
    mask = None
    if sparse:
        assert bits == 4 and K % 32 == 0
        # exactly 16 of every 32 rows kept, uniformly at random per (block, column)
        r = rng.random((K // 32, 32, S), dtype=np.float32)
        order = np.argsort(r, axis=1)
        keep = np.zeros((K // 32, 32, S), dtype=bool)
        np.put_along_axis(keep, order[:, :16, :], True, axis=1)
        keep = keep.reshape(K, S)
        matrix, mask = sparse_pack(np.ascontiguousarray(codes.T),
                                   np.ascontiguousarray(keep.T).astype(np.uint8))
        codes = np.where(keep, codes, np.uint8(0))
    else:
        matrix = pack_dense(bits, codes)
    return dict(K=K, S=S, M=M, B=B, bits=bits, group_size=group_size, states=states,
                codes=codes, matrix=matrix, sparse_mask=mask, keep=keep,
                scales=scales, zeros=zeros)
