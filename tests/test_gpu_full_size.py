"""The benchmark configurations at their full sizes against the oracle (seed 0,
the distributions the configurations state): K=20480 x S=5120 matvec, the 16:32
matvec at K=S=16384 (g=64) and matmul at M=2048, K=5120, S=20480 (g=64), int3 and
int2 at K=5120, S=20480 for M=1 and M=2048.  Matvecs are checked on every output,
matmuls on 24 sampled rows.  (K=5120 x S=20480 int4 at M=1 and M=2048 is in
test_gpu_products.py.)  These shapes take launch paths no small case reaches: strips
of 64 columns with many K splits, the split of a half-empty last round of tiles with
the int3 / int2 / 16:32 decoders, 640-tile grids."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    from tests import helpers
    return helpers


def _matvec_against_oracle_by_column_chunks(H, p, got, chunk=2048):
    """every output of a matvec: exact product on the fp16 weights and fp32 dequantise-then-matmul,
    computed a slab of columns at a time (the dequantised matrix of the largest shape is 1 GB in fp32)"""
    K, S, bits, g = p["K"], p["S"], p["bits"], p["group_size"]
    x = p["states"].reshape(1, K)
    exact = np.empty((1, S), np.float64)
    f32 = np.empty((1, S), np.float32)
    for c0 in range(0, S, chunk):
        cols = slice(c0, min(S, c0 + chunk))
        mask = None if p["sparse_mask"] is None else p["sparse_mask"][:, cols]
        w16 = O.dequantize_matrix(bits, p["matrix"][:, cols], p["scales"][:, cols], p["zeros"][:, cols], g, mask)
        exact[:, cols] = O.matmul_exact(x, w16)
        w32 = O.dequantize_matrix_fp32(bits, p["matrix"][:, cols], p["scales"][:, cols], p["zeros"][:, cols], g, mask)
        f32[:, cols] = O.matmul_fp32(x, w32)
    f32 = f32.view(H.OracleArray)
    f32.bits = bits                                           # (the tight-floor bar depends on the format)
    H.assert_product_close(got.reshape(1, 1, S), exact.reshape(1, 1, S), f32.reshape(1, 1, S))


def _matmul_rows_against_oracle(H, p, out, rows):
    bits, g = p["bits"], p["group_size"]
    xs = p["states"][0, rows]
    w16 = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], g, p["sparse_mask"])
    assert O.max_rel_error(O.matmul_exact(xs, w16), out[0, rows], floor_frac=H.FLOOR_EXACT_MTX) < H.TOL_EXACT_MTX
    del w16
    w32 = O.dequantize_matrix_fp32(bits, p["matrix"], p["scales"], p["zeros"], g, p["sparse_mask"])
    assert O.max_rel_error(O.matmul_fp32(xs, w32), out[0, rows]) < H.TOL_F32
    assert np.all(np.isfinite(out.astype(np.float32)))


def test_int4_matvec_transposed_shape(H):
    p = O.make_problem(K=20480, S=5120, M=1, bits=4, group_size=128, seed=0)
    d = H.dev_problem(p)
    _matvec_against_oracle_by_column_chunks(H, p, H.run_capi(p, d, "vec"))
    _matvec_against_oracle_by_column_chunks(H, p, H.run_ext(p, d))


@pytest.mark.parametrize("bits,zero", [(3, 3.5), (2, 1.5)])
def test_int3_int2_matvec_and_matmul(H, bits, zero):
    K, S, g, M = 5120, 20480, 128, 2048
    p = O.make_problem(K=K, S=S, M=1, bits=bits, group_size=g, seed=0, scale_range=(0.004, 0.08), zero_const=zero)
    d = H.dev_problem(p)
    _matvec_against_oracle_by_column_chunks(H, p, H.run_capi(p, d, "vec"))
    xs = np.random.default_rng(5).standard_normal((1, M, K), dtype=np.float32).astype(np.float16)
    pm = dict(p, M=M, states=xs)
    out = H.run_capi(pm, H.dev_problem(pm), "mtx")
    _matmul_rows_against_oracle(H, pm, out, np.linspace(0, M - 1, 24).astype(int))


def test_sparse_matmul_full_size(H):
    K, S, g, M = 5120, 20480, 64, 2048
    p = O.make_problem(K=K, S=S, M=M, bits=4, group_size=g, sparse=True, seed=0)
    out = H.run_capi(p, H.dev_problem(p), "mtx")
    _matmul_rows_against_oracle(H, p, out, np.linspace(0, M - 1, 24).astype(int))


def test_sparse_matvec_full_size(H):
    """K = S = 16384, g = 64.  The 16-of-32 masks are drawn per (block, column) from 4096 random
    subsets (as the reference's harness draws from 1024, kernel_test.py:200-220); the packed
    operands come from the device packer (bit-exact against the oracle's in test_gpu_formats.py)
    and the expected values straight from the unpacked codes and mask, so the check does not
    depend on any unpack."""
    K = S = 16384
    g = 64
    rng = np.random.default_rng(0)
    table = np.zeros(4096, np.uint32)
    for i in range(4096):
        table[i] = np.bitwise_or.reduce(np.uint32(1) << rng.choice(32, 16, replace=False).astype(np.uint32))
    words = table[rng.integers(0, 4096, size=(K // 32, S))]                        # [K/32, S]
    keep = ((words[:, None, :] >> np.arange(32, dtype=np.uint32)[None, :, None]) & 1).astype(bool).reshape(K, S)
    codes = rng.integers(0, 16, size=(K, S), dtype=np.uint8)
    scales = rng.uniform(0.001, 0.02, size=(K // g, S)).astype(np.float16)
    zeros = rng.uniform(0.0, 15.0, size=(K // g, S)).astype(np.float16)
    x = rng.standard_normal((1, 1, K), dtype=np.float32).astype(np.float16)
    dev = "cuda"
    wt = torch.empty((K // 16, S), dtype=torch.int32, device=dev)
    mk = torch.empty((K // 32, S), dtype=torch.int32, device=dev)
    bad = torch.zeros(1, dtype=torch.int32, device=dev)
    H.capi.sparse_pack(wt, mk, torch.from_numpy(np.ascontiguousarray(codes.T)).to(dev),
                       torch.from_numpy(np.ascontiguousarray(keep.T).astype(np.uint8)).to(dev), bad)
    assert int(bad.item()) == 0
    assert np.array_equal(mk.cpu().numpy().view(np.uint32), words)
    outs = torch.zeros((1, 1, S), dtype=torch.float16, device=dev)
    ws = H.capi.new_workspace(S)
    H.capi.matvec(4, outs, wt, H.t(x), H.t(scales), H.t(zeros), g, mk, ws)
    torch.cuda.synchronize()
    got = outs.cpu().numpy()
    exact = np.empty((1, S), np.float64)
    f32 = np.empty((1, S), np.float32)
    gi = np.arange(K) // g
    for c0 in range(0, S, 2048):
        cols = slice(c0, c0 + 2048)
        q = codes[:, cols]
        s, z = scales[gi][:, cols], zeros[gi][:, cols]
        w16 = np.where(keep[:, cols], O.dequant_linear(q, s, z), np.float16(0))
        exact[:, cols] = O.matmul_exact(x.reshape(1, K), w16)
        w32 = np.where(keep[:, cols], (q.astype(np.float32) - z.astype(np.float32)) * s.astype(np.float32), np.float32(0))
        f32[:, cols] = O.matmul_fp32(x.reshape(1, K), w32)
    H.assert_product_close(got, exact.reshape(1, 1, S), f32.reshape(1, 1, S))


@pytest.mark.parametrize("bits", [4, 3])
def test_mixed_quantisation_modes_matmul_full_size(H, bits):
    """M = 2048, K = 5120, S = 20480 with exponent-mode groups scattered over the matrix (negative scale:
    matmul.cuh:414-428): one whole group row, every third column of another, single entries elsewhere.
    Every 256 x 256 tile then contains both modes and takes the pipelined loop whose decode serves either."""
    K, S, g, M = 5120, 20480, 128, 2048
    p = O.make_problem(K=K, S=S, M=M, bits=bits, group_size=g, seed=3, zero_range=(0.0, 4.0))
    sc = p["scales"].copy()
    sc[7] = -sc[7]
    sc[19, ::3] = -sc[19, ::3]
    sc[np.arange(40), np.arange(40) * 509 % S] *= np.float16(-1)
    p = dict(p, scales=sc)
    out = H.run_capi(p, H.dev_problem(p), "mtx")
    rows = np.linspace(0, M - 1, 24).astype(int)
    # (the fp32 dequantise-then-matmul oracle is linear-mode only: the exact product on the fp16 weights is the check)
    w16 = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], g, None)
    assert O.max_rel_error(O.matmul_exact(p["states"][0, rows], w16), out[0, rows], floor_frac=H.FLOOR_EXACT_MTX) < H.TOL_EXACT_MTX
    assert np.all(np.isfinite(out.astype(np.float32)))


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_mixed_quantisation_modes_matvec_full_size(H, bits):
    """K = 5120, S = 20480, M = 1 with exponent-mode groups: one whole group row, every third column of another,
    single entries elsewhere.  The matvec's first pass skips those (group, column) pairs; its second pass visits
    only the units that hold any and decodes them with the exponent form of the same operands."""
    K, S, g = 5120, 20480, 128
    kw = {} if bits == 4 else dict(scale_range=(0.004, 0.08), zero_const=3.5 if bits == 3 else 1.5)
    p = O.make_problem(K=K, S=S, M=1, bits=bits, group_size=g, seed=4, **kw)
    sc = p["scales"].copy()
    sc[7] = -sc[7]
    sc[19, ::3] = -sc[19, ::3]
    sc[np.arange(40), np.arange(40) * 509 % S] *= np.float16(-1)
    p = dict(p, scales=sc)
    got = H.run_capi(p, H.dev_problem(p), "vec")
    x = p["states"].reshape(1, K)
    exact = np.empty((1, S), np.float64)
    for c0 in range(0, S, 2048):
        cols = slice(c0, c0 + 2048)
        w16 = O.dequantize_matrix(bits, p["matrix"][:, cols], sc[:, cols], p["zeros"][:, cols], g, None)
        exact[:, cols] = O.matmul_exact(x, w16)
    exact = exact.reshape(1, 1, S)
    H.assert_product_close(got, exact, exact.astype(np.float32))


@pytest.mark.parametrize("bits", [4, 3])
def test_long_k_narrow_output_takes_split_small_tiles(H, bits):
    """K=14336, S=4096, 1152 rows: nine rows of 128 x 256 tiles would fill the GPU once; the long K makes
    256 x 128 tiles split three ways along K the faster choice.  Sampled rows against the oracle, the whole
    output against the unsplit kernel."""
    K, S, g, M = 14336, 4096, 128, 1152
    tiles = H.capi.describe_launch("mtx", bits, 1, M, K, S, g)
    assert "tile=256x128,plain> tiles=160 ksplit=3" in tiles, tiles
    kw = {} if bits == 4 else dict(scale_range=(0.004, 0.08), zero_const=3.5)
    p = O.make_problem(K=K, S=S, M=1, bits=bits, group_size=g, seed=3, **kw)
    xs = np.random.default_rng(6).standard_normal((1, M, K), dtype=np.float32).astype(np.float16)
    pm = dict(p, M=M, states=xs)
    d = H.dev_problem(pm)
    out = H.run_capi(pm, d, "mtx", outs_init=np.full((1, M, S), 5.0, np.float16))
    _matmul_rows_against_oracle(H, pm, out, np.array([0, 1, 127, 128, 255, 256, 511, 512, 767, 1023, 1024, 1150, 1151]))
    H.capi.tune(6, 1)
    try:
        ref = H.run_capi(pm, d, "mtx")
    finally:
        H.capi.tune(6, 0)
    assert O.max_rel_error(ref.astype(np.float64), out) < H.TOL_EXACT_MTX
