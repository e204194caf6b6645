"""GPU parity, floating-point side: matvec and matmul against the CPU oracle
within the tolerances stated in tests/helpers.py, through the C ABI and through
the ``int4matmul`` extension."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

FORMATS = [(4, False), (3, False), (2, False), (4, True)]


@pytest.fixture(scope="module")
def H():
    from tests import helpers
    return helpers


def _problem(bits, sparse, **kw):
    if bits != 4:       # int3 / int2 benchmark configuration: scales U(0.004, 0.08), zero at the mid-code
        kw.setdefault("scale_range", (0.004, 0.08))
        kw.setdefault("zero_const", 3.5 if bits == 3 else 1.5)
    return O.make_problem(bits=bits, sparse=sparse, **kw)


# ------------------------------------------------------------------- matvec
@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("K,S,g", [(1024, 1024, 64), (64, 64, 64), (2048, 320, 128), (5120, 256, -1)])
def test_matvec_parity(H, bits, sparse, K, S, g):
    p = _problem(bits, sparse, K=K, S=S, M=1, group_size=g, seed=0)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "vec")
    H.assert_product_close(got, exact, f32)
    got2 = H.run_ext(p, d)
    H.assert_product_close(got2, exact, f32)


@pytest.mark.parametrize("bits,sparse,g", [(4, False, 128), (3, False, 256), (4, True, 64), (2, False, -1)])
def test_matvec_of_a_k_longer_than_one_launch_covers(H, bits, sparse, g):
    """K = 458752 + 8192: beyond the 32 x 224 units of 64 rows that one launch stages and splits, so the
    product runs as two launches, the second adding onto the first (the reference's grid covers any K:
    matvec_kernel.cu:339-347); with a prior in outs and two batch rows"""
    K = 458752 + 8192
    p = _problem(bits, sparse, K=K, S=64, M=1, B=2, group_size=g, seed=21)
    d = H.dev_problem(p)
    assert H.capi.describe_launch("vec", bits, 1, 1, K, 64, g, sparse).count("matvec_kernel<") == 2
    exact, f32 = H.oracles(p)
    prior = np.random.default_rng(2).standard_normal((2, 1, 64)).astype(np.float16)
    H.capi.tune(5, 1)                    # (the single-row kernel, not the few-row kernel the batch would take)
    try:
        got = H.run_capi(p, d, "vec", outs_init=prior)
    finally:
        H.capi.tune(5, 0)
    H.assert_product_close(got, exact, f32, prior=prior)


@pytest.mark.parametrize("bits,sparse", FORMATS)
def test_matvec_accumulates_onto_prior_outs_and_batches(H, bits, sparse):
    p = _problem(bits, sparse, K=512, S=192, M=1, B=3, group_size=64, seed=4)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    prior = np.random.default_rng(1).standard_normal((3, 1, 192)).astype(np.float16)
    got = H.run_capi(p, d, "vec", outs_init=prior)
    H.assert_product_close(got, exact, f32, prior=prior)
    # closed form of the quirk: fp16(fp32(prior) + y); y is within tolerance of exact
    want = O.matvec_expected(prior, exact)
    assert O.max_rel_error(want, got) < H.TOL_EXACT


@pytest.mark.parametrize("bits,sparse", FORMATS)
def test_matvec_exponent_mode_columns(H, bits, sparse):
    p = _problem(bits, sparse, K=512, S=256, M=1, group_size=128, seed=9)
    p["scales"][:, 1::4] *= np.float16(-1)      # exponent mode in a quarter of the columns
    p["scales"][2, :] *= np.float16(-1)         # and flipped for one whole group
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    for kind in ("vec", "mtx"):
        got = H.run_capi(p, d, kind)
        # (a single row through the matmul entry is served by the matvec kernel: the matvec's class)
        H.assert_product_close(got, exact, f32, kind="vec" if kind == "vec" else H.matmul_kind(p))


@pytest.mark.parametrize("bits,sparse", FORMATS)
def test_matvec_exponent_mode_groups_split_k(H, bits, sparse):
    """K = 8192 split over several workgroups, 64-row groups: exponent mode in whole groups, in every third column of
    another and in single (group, column) pairs -- the second pass over the units that hold any, for 16:32 with the
    kept codes expanded as in the first pass and their halves turned into +-2^e"""
    K, S, g = 8192, 2048, 64
    p = _problem(bits, sparse, K=K, S=S, M=1, group_size=g, seed=11)
    assert "splits=" in H.capi.describe_launch("vec", bits, 1, 1, K, S, g, sparse)
    sc = p["scales"]
    sc[5] *= np.float16(-1)
    sc[77, ::3] *= np.float16(-1)
    sc[np.arange(128), np.arange(128) * 37 % S] *= np.float16(-1)
    exact, f32 = H.oracles(p)
    prior = np.random.default_rng(3).standard_normal((1, 1, S)).astype(np.float16)
    got = H.run_capi(p, H.dev_problem(p), "vec", outs_init=prior)
    H.assert_product_close(got, exact, f32, prior=prior)


@pytest.mark.parametrize("bits,sparse,K", [(4, False, 5120), (3, False, 1024), (2, False, 2048),
                                           (4, True, 16384)])
def test_degenerate_known_answer(H, bits, sparse, K):
    """all-ones codes and states, zero zero-points, unit scales: every output is
    K (K/2 with 16:32 sparsity), exactly -- kernel_test.py:187-192,210-215,242-243"""
    S = 256
    codes = np.ones((K, S), np.uint8)
    if sparse:
        keep = np.zeros((S, K // 32, 32), np.uint8)
        keep[:, :, 16:] = 1
        matrix, mask = O.sparse_pack(np.ascontiguousarray(codes.T), keep.reshape(S, K))
    else:
        matrix, mask = O.pack_dense(bits, codes), None
    p = dict(B=1, S=S, K=K, bits=bits, group_size=128, matrix=matrix, sparse_mask=mask,
             states=np.ones((1, 1, K), np.float16), scales=np.ones((K // 128, S), np.float16),
             zeros=np.zeros((K // 128, S), np.float16))
    want = K // 2 if sparse else K
    for M, kind in ((1, "vec"), (1, "mtx"), (70, "mtx")):
        p["M"] = M
        p["states"] = np.ones((1, M, K), np.float16)
        got = H.run_capi(p, H.dev_problem(p), kind)
        assert np.all(got.astype(np.float64) == want), (M, kind)


# ------------------------------------------------------------------- matmul
@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("M,K,S,g", [(2048, 128, 128, 128), (70, 256, 192, 64), (1, 512, 64, 128), (500, 192, 256, 64),
                                     (257, 1024, 320, -1), (342, 256, 512, 64), (400, 320, 256, 64), (600, 128, 384, 128),
                                     (700, 192, 256, 64)])
def test_matmul_parity(H, bits, sparse, M, K, S, g):
    p = _problem(bits, sparse, K=K, S=S, M=M, group_size=g, seed=M)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx")
    H.assert_product_close(got, exact, f32, kind=H.matmul_kind(p))


@pytest.mark.parametrize("bits,sparse", FORMATS)
def test_matmul_overwrites_outs_batches_and_matches_matvec(H, bits, sparse):
    p = _problem(bits, sparse, K=256, S=128, M=5, B=2, group_size=64, seed=3)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    junk = np.full((2, 5, 128), 123.0, np.float16)
    got = H.run_capi(p, d, "mtx", outs_init=junk)           # prior contents must not leak in
    H.assert_product_close(got, exact, f32, kind=H.matmul_kind(p))
    # M == 1 through the forced-matmul entry point agrees with the matvec entry point
    q = _problem(bits, sparse, K=256, S=128, M=1, group_size=64, seed=3)
    dq = H.dev_problem(q)
    a = H.run_ext(q, dq, fn_name=f"quant_int{bits}_linear_mult_mtx")
    b = H.run_ext(q, dq, fn_name=f"quant_int{bits}_linear_mult_vec")
    c = H.run_ext(q, dq, fn_name=f"quant_int{bits}_linear_mult")
    assert O.max_rel_error(a.astype(np.float64), b) < H.TOL_EXACT
    assert np.array_equal(b, c)                              # auto-dispatch takes the matvec


# ----------------------------------------------------------- extension API
def test_extension_argument_errors(H):
    ext = H.pkg.load_extension()
    p = O.make_problem(K=128, S=64, M=1, bits=4, group_size=64, seed=0)
    d = H.dev_problem(p)
    outs = torch.zeros((1, 1, 64), dtype=torch.float16, device=H.DEV)
    ok = (outs, d["matrix"], d["states"], d["scales"], d["zeros"], 64, None)
    ext.quant_matmul(4, *ok)
    with pytest.raises(ValueError):
        ext.quant_matmul(5, *ok)
    with pytest.raises(RuntimeError):                       # group size not a multiple of 64
        ext.quant_matmul(4, outs, d["matrix"], d["states"], d["scales"], d["zeros"], 32, None)
    with pytest.raises(RuntimeError):                       # wrong dtype
        ext.quant_matmul(4, outs.float(), d["matrix"], d["states"], d["scales"], d["zeros"], 64, None)
    with pytest.raises(RuntimeError):                       # packed rows do not match in_size
        ext.quant_matmul(4, outs, d["matrix"][:8], d["states"], d["scales"], d["zeros"], 64, None)
    with pytest.raises(RuntimeError):                       # sparsity with int3
        m3 = torch.zeros((12, 64), dtype=torch.int32, device=H.DEV)
        msk = torch.zeros((6, 64), dtype=torch.int32, device=H.DEV)
        ext.quant_matmul(3, outs, m3, d["states"], d["scales"], d["zeros"], 64, msk)
    with pytest.raises(RuntimeError):                       # _vec entry point with M != 1
        x2 = torch.zeros((1, 2, 128), dtype=torch.float16, device=H.DEV)
        o2 = torch.zeros((1, 2, 64), dtype=torch.float16, device=H.DEV)
        ext.quant_int4_linear_mult_vec(o2, d["matrix"], x2, d["scales"], d["zeros"], 64, None)


def test_single_group_accepts_1d_scales(H):
    p = O.make_problem(K=256, S=128, M=1, bits=4, group_size=-1, seed=8)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    ext = H.pkg.load_extension()
    for M in (1, 9):
        x = torch.from_numpy(np.tile(p["states"], (1, M, 1))).to(H.DEV)
        outs = torch.zeros((1, M, 128), dtype=torch.float16, device=H.DEV)
        ext.quant_matmul(4, outs, d["matrix"], x, d["scales"][0], d["zeros"][0], -1, None)
        got = outs.cpu().numpy()
        for m in range(M):
            H.assert_product_close(got[:, m:m + 1], exact, f32, kind="vec")    # (9 rows: the few-row kernel)


# ------------------------------------------------- full-size benchmark shapes
def test_full_size_matvec_and_matmul_c2_c3(H):
    """K=5120, S=20480, g=128 (the headline matvec and matmul shapes): the matvec against the
    oracle on every output; the M=2048 matmul on 24 sampled rows against the
    oracle, plus row-linearity of the whole product (a size-independent
    property: the product of a sum of two row blocks equals the sum of products
    within fp16 rounding)."""
    K, S, g = 5120, 20480, 128
    p = O.make_problem(K=K, S=S, M=1, bits=4, group_size=g, seed=0)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "vec")
    H.assert_product_close(got, exact, f32)
    # exponent mode in some columns takes the kernels' general loops at full size
    M = 2048
    rng = np.random.default_rng(5)
    xs = rng.standard_normal((1, M, K), dtype=np.float32).astype(np.float16)
    pm = dict(p, M=M, states=xs)
    dm = H.dev_problem(pm)
    out = H.run_capi(pm, dm, "mtx")
    rows = np.linspace(0, M - 1, 24).astype(int)
    w16 = O.dequantize_matrix(4, p["matrix"], p["scales"], p["zeros"], g)
    want = O.matmul_exact(xs[0, rows], w16)
    assert O.max_rel_error(want, out[0, rows], floor_frac=H.FLOOR_EXACT_MTX) < H.TOL_EXACT_MTX
    w32 = O.dequantize_matrix_fp32(4, p["matrix"], p["scales"], p["zeros"], g)
    assert O.max_rel_error(O.matmul_fp32(xs[0, rows], w32), out[0, rows]) < H.TOL_F32
    # M = 1 through the matmul kernel agrees with the matvec kernel
    one = H.run_capi(p, d, "mtx")
    assert O.max_rel_error(got.astype(np.float64), one) < H.TOL_EXACT


@pytest.mark.parametrize("bits,sparse,variant", [(4, False, 5), (3, False, 5), (2, False, 5), (4, False, 6),
                                                 (3, False, 6), (2, False, 6), (4, True, 6), (4, False, 9),
                                                 (3, False, 9), (2, False, 9)])
@pytest.mark.parametrize("M,K,S,g,B", [(256, 512, 512, 128, 1), (512, 192, 256, 64, 2), (256, 2048, 256, -1, 1),
                                       (512, 448, 512, 64, 1)])
def test_pipelined_matmul_with_exponent_groups(H, bits, sparse, variant, M, K, S, g, B):
    """tile-aligned dense shapes take the pipelined kernel (variant 5: 256 x 128
    tiles, variant 6: 256 x 256 with the two halves of the workgroup in opposite
    phases for the dense formats, variant 9: 256 x 256 in the plain order); negative
    scales in a few columns force its general loop for the tiles that contain them.
    K = 192 is six K steps (one trip of the unrolled loop), K = 448 fourteen (two trips
    and a remainder), K = 2048 with a single group runs many trips."""
    from int4matmul_kernels_amd import capi
    p = O.make_problem(K=K, S=S, M=M, bits=bits, group_size=g, sparse=sparse, seed=21 + bits, B=B)
    capi.tune(3, variant)
    try:
        d = H.dev_problem(p)
        exact, f32 = H.oracles(p)
        H.assert_product_close(H.run_capi(p, d, "mtx"), exact, f32, kind="mtx")
        sc = p["scales"].reshape(-1, S)
        sc[sc.shape[0] // 2, 200:210] *= np.float16(-1)
        d = H.dev_problem(p)
        exact, f32 = H.oracles(p)
        H.assert_product_close(H.run_capi(p, d, "mtx"), exact, f32, kind="mtx")
    finally:
        capi.tune(3, 0)


# ---- 257 ... 384 rows: three rows of 128 x 256 tiles of the pipelined kernel (tuning key 3 = 7 forces them), and the
# padded 256-row tiles that serve 257 ... 341 rows on small grids and for 16:32
@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("M,K,S,g", [(384, 512, 512, 128), (300, 2048, 256, 64), (257, 1024, 768, -1), (341, 2560, 256, 128)])
def test_matmul_three_rows_of_128_row_tiles(H, bits, sparse, M, K, S, g):
    p = _problem(bits, sparse, K=K, S=S, M=M, group_size=g, seed=M + S)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    H.capi.tune(8, 1)            # (not the few-row path)
    try:
        auto = H.run_capi(p, d, "mtx", outs_init=np.full((1, M, S), 4.0, np.float16))
        H.assert_product_close(auto, exact, f32, kind="mtx")
        H.capi.tune(3, 7)
        try:
            got = H.run_capi(p, d, "mtx", outs_init=np.full((1, M, S), 4.0, np.float16))
        finally:
            H.capi.tune(3, 0)
    finally:
        H.capi.tune(8, 0)
    H.assert_product_close(got, exact, f32, kind="mtx")
    assert O.max_rel_error(auto.astype(np.float64), got) < H.TOL_EXACT_MTX


@pytest.mark.parametrize("bits,sparse", [(4, False), (4, True)])
def test_matmul_three_rows_default_rule_and_exponent_groups(H, bits, sparse):
    """M=300 against S=11264 (44 tile columns: 132 tiles of 128 x 256) takes the variant by default for the dense
    format; some exponent-mode groups on top"""
    p = _problem(bits, sparse, K=1024, S=11264, M=300, group_size=128, seed=12)
    p["scales"][2, 100:108] *= np.float16(-1)
    p["scales"][5, 7000] *= np.float16(-1)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    H.capi.tune(8, 1)
    try:
        got = H.run_capi(p, d, "mtx")
    finally:
        H.capi.tune(8, 0)
    H.assert_product_close(got, exact, f32, kind="mtx")


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (4, True)])
def test_matmul_five_rows_of_128_row_tiles_default_rule(H, bits, sparse):
    """M=600 (five tile rows of 128) against S=11264: 220 tiles of 128 x 256, taken by default"""
    p = _problem(bits, sparse, K=512, S=11264, M=600, group_size=64, seed=15)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((1, 600, 11264), 4.0, np.float16))
    H.assert_product_close(got, exact, f32, kind="mtx")


@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("B,M,K,S", [(5, 130, 512, 512), (32, 20, 256, 1024), (3, 300, 320, 256), (2, 600, 1024, 384)])
def test_batches_are_one_product_of_all_their_rows(H, bits, sparse, B, M, K, S):
    """[B, M, K] states and [B, M, S] outputs are contiguous, so B products of M rows run as one product of B * M rows:
    the same bits as the flattened call, and the oracle's values"""
    capi = H.capi
    assert capi.describe_launch("mtx", bits, B, M, K, S, 64, sparse) == capi.describe_launch("mtx", bits, 1, B * M, K, S, 64, sparse)
    p = _problem(bits, sparse, K=K, S=S, M=M, B=B, group_size=64, seed=B + M)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((B, M, S), 6.0, np.float16))
    H.assert_product_close(got, exact, f32, kind=H.matmul_kind(p))
    flat = torch.full((1, B * M, S), 6.0, dtype=torch.float16, device="cuda")
    ws = capi.new_matmul_workspace(1, B * M, K, S, sparse)
    capi.matmul(bits, flat, d["matrix"], d["states"].reshape(1, B * M, K), d["scales"], d["zeros"], 64, d["mask"], ws)
    torch.cuda.synchronize()
    assert np.array_equal(got.reshape(B * M, S), flat.cpu().numpy().reshape(B * M, S))
