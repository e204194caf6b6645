"""The few-row kernels (2 .. 96 rows of states in all, on suitable shapes up to 512; dense
formats and 16:32 sparse int4): every packed word is read once for all rows.  It serves `quant_matmul` with small M (any
batch layout that flattens to <= 32 rows) and the matvec entry with B > 1.
Its numerics are the matvec's (exact sum of x (q - z) s, no per-weight fp16
rounding), so the matvec tolerance applies; it is also checked against the
general kernels it replaces (tuning key 5 switches it off)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402


@pytest.fixture(scope="module")
def H():
    from tests import helpers
    return helpers


def _check(H, p, kind, prior=None):
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, kind, outs_init=prior)
    # the kernels that apply scale and zero in fp32 per group are also held to the fp32 oracle on the tight
    # floor; which kernel serves the call is the launcher's word (it sees this thread's tuning keys too)
    line = H.capi.describe_launch(kind, p["bits"], p["B"], p["M"], p["K"], p["S"], p["group_size"], p["sparse_mask"] is not None)
    tight = line.startswith(("skinny_kernel", "matvec_kernel"))
    H.assert_product_close(got, exact, f32, prior=prior if kind == "vec" else None, kind="vec", tight=tight)
    return d, got


def _problem(bits, **kw):
    if bits != 4:       # scales U(0.004, 0.08), zero at the mid-code
        kw.setdefault("scale_range", (0.004, 0.08))
        kw.setdefault("zero_const", 3.5 if bits == 3 else 1.5)
    return O.make_problem(bits=bits, **kw)


@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("M", [2, 3, 8, 9, 16, 17, 31, 32, 33, 64, 71, 96])
@pytest.mark.parametrize("K,S,g", [(512, 256, 128), (64, 64, 64), (1024, 192, -1), (320, 1024, 64), (256, 8192, 128)])
def test_few_rows_matmul(H, bits, M, K, S, g):
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=M + K)
    junk = np.full((1, M, S), -77.0, np.float16)
    d, got = _check(H, p, "mtx", prior=junk)                      # matmul semantics: prior contents overwritten
    # against the general kernel it replaces
    H.capi.tune(5, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        H.capi.tune(5, 0)
    assert O.max_rel_error(ref.astype(np.float64), got) < H.TOL_EXACT


@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("B,M", [(2, 1), (5, 1), (32, 1), (4, 4), (3, 7), (40, 1), (5, 17), (96, 1)])
def test_few_rows_batches_flatten(H, bits, B, M):
    p = _problem(bits, K=768, S=320, M=M, group_size=128, seed=B * 10 + M, B=B)
    _check(H, p, "mtx")
    if M == 1:
        # the matvec entry adds onto the prior contents of outs
        prior = np.random.default_rng(B).standard_normal((B, 1, 320)).astype(np.float16)
        _check(H, p, "vec", prior=prior)


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_few_rows_exponent_mode_columns(H, bits):
    p = _problem(bits, K=512, S=256, M=6, group_size=128, seed=9)
    p["scales"][1, 40:48] *= np.float16(-1)                   # one strip switches to the exact decode
    p["scales"][3, 200] *= np.float16(-1)
    _check(H, p, "mtx")


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_few_rows_degenerate_known_answer(H, bits):
    K, S, M = 1024, 128, 12
    codes = np.ones((K, S), np.uint8)
    p = dict(B=1, M=M, S=S, K=K, bits=bits, group_size=128, matrix=O.pack_dense(bits, codes), sparse_mask=None,
             states=np.ones((1, M, K), np.float16), scales=np.ones((K // 128, S), np.float16),
             zeros=np.zeros((K // 128, S), np.float16))
    got = H.run_capi(p, H.dev_problem(p), "mtx")
    assert np.all(got.astype(np.float64) == K)


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_few_rows_full_size(H, bits):
    """K=5120, S=20480, 16 rows: the whole output against the oracle"""
    p = _problem(bits, K=5120, S=20480, M=16, group_size=128, seed=4)
    _check(H, p, "mtx")


# ---- 16:32 sparse int4 through the same kernel
@pytest.mark.parametrize("M", [2, 3, 8, 9, 16, 17, 32, 33, 64, 96])
@pytest.mark.parametrize("K,S,g", [(512, 256, 64), (64, 64, 64), (1024, 192, -1), (320, 1024, 64), (256, 8192, 128)])
def test_few_rows_sparse_matmul(H, M, K, S, g):
    p = O.make_problem(bits=4, K=K, S=S, M=M, group_size=g, sparse=True, seed=M + K)
    junk = np.full((1, M, S), -77.0, np.float16)
    d, got = _check(H, p, "mtx", prior=junk)
    H.capi.tune(5, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        H.capi.tune(5, 0)
    assert O.max_rel_error(ref.astype(np.float64), got) < H.TOL_EXACT


@pytest.mark.parametrize("B,M", [(2, 1), (5, 1), (32, 1), (4, 4), (3, 7), (40, 1), (96, 1)])
def test_few_rows_sparse_batches_flatten(H, B, M):
    p = O.make_problem(bits=4, K=768, S=320, M=M, group_size=64, sparse=True, seed=B * 10 + M, B=B)
    _check(H, p, "mtx")
    if M == 1:
        prior = np.random.default_rng(B).standard_normal((B, 1, 320)).astype(np.float16)
        _check(H, p, "vec", prior=prior)


def test_few_rows_sparse_exponent_mode_columns(H):
    p = O.make_problem(bits=4, K=512, S=256, M=6, group_size=64, sparse=True, seed=9)
    p["scales"][1, 40:48] *= np.float16(-1)
    p["scales"][3, 200] *= np.float16(-1)
    _check(H, p, "mtx")


def test_few_rows_sparse_crowded_masks(H):
    """masks whose kept rows crowd one end of the block: all 16 codes lie before, or
    after, some 8-row chunk"""
    K, S, M = 256, 64, 5
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 16, size=(K, S), dtype=np.uint8)
    keep = np.zeros((K // 32, 32, S), dtype=bool)
    keep[0, :16] = True                      # first half
    keep[1, 16:] = True                      # second half
    keep[2, 8:24] = True                     # the middle
    keep[3, ::2] = True                      # every other row
    keep[4, :8] = True
    keep[4, 24:] = True                      # both ends
    keep[5, 1::2] = True
    keep[6, :4] = True
    keep[6, 20:] = True
    keep[7, 3:19] = True
    keep = keep.reshape(K, S)
    matrix, mask = O.sparse_pack(np.ascontiguousarray(codes.T), np.ascontiguousarray(keep.T).astype(np.uint8))
    G = K // 64
    p = dict(B=1, M=M, S=S, K=K, bits=4, group_size=64, matrix=matrix, sparse_mask=mask, keep=keep,
             codes=np.where(keep, codes, np.uint8(0)), states=rng.standard_normal((1, M, K)).astype(np.float16),
             scales=rng.uniform(0.001, 0.02, size=(G, S)).astype(np.float16),
             zeros=rng.uniform(0, 15, size=(G, S)).astype(np.float16))
    _check(H, p, "mtx")
    _check(H, dict(p, M=1, states=p["states"][:, :1]), "vec")


def test_few_rows_sparse_degenerate_known_answer(H):
    K, S, M = 1024, 128, 12
    codes = np.ones((S, K), np.uint8)
    keep = np.zeros((S, K), np.uint8)
    keep[:, ::2] = 1
    matrix, mask = O.sparse_pack(codes, keep)
    p = dict(B=1, M=M, S=S, K=K, bits=4, group_size=64, matrix=matrix, sparse_mask=mask,
             states=np.ones((1, M, K), np.float16), scales=np.ones((K // 64, S), np.float16),
             zeros=np.zeros((K // 64, S), np.float16))
    got = H.run_capi(p, H.dev_problem(p), "mtx")
    assert np.all(got.astype(np.float64) == K // 2)


def test_few_rows_sparse_full_size(H):
    p = O.make_problem(bits=4, K=5120, S=20480, M=8, group_size=64, sparse=True, seed=4)
    _check(H, p, "mtx")


# ---- long K against a narrow matrix: the strips are split along K across workgroups
@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (2, False), (4, True)])
@pytest.mark.parametrize("M,K,S,g", [(8, 16384, 256, 128), (40, 8192, 128, 64), (2, 12288, 512, -1), (17, 6144, 192, 128)])
def test_few_rows_split_k(H, bits, sparse, M, K, S, g):
    capi = H.capi
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=M + S, sparse=sparse)
    assert capi.matmul_workspace_bytes(1, M, K, S, sparse) > capi.lib().int4mm_workspace_bytes(S), "shape should split"
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    outs = []
    ws = capi.new_matmul_workspace(1, M, K, S, sparse)
    for _ in range(3):                                   # one workspace: the counters must come back to zero
        o = torch.full((1, M, S), -5.0, dtype=torch.float16, device="cuda")
        capi.matmul(bits, o, d["matrix"], d["states"], d["scales"], d["zeros"], g, d["mask"], ws)
        torch.cuda.synchronize()
        outs.append(o.cpu().numpy())
    H.assert_product_close(outs[0], exact, f32, kind="vec")
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    capi.tune(6, 1)                                      # unsplit
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        capi.tune(6, 0)
    assert O.max_rel_error(ref.astype(np.float64), outs[0]) < H.TOL_EXACT


def test_few_rows_split_k_matvec_entry_accumulates(H):
    p = _problem(4, K=16384, S=256, M=1, B=6, group_size=128, seed=77)
    prior = np.random.default_rng(1).standard_normal((6, 1, 256)).astype(np.float16)
    _check(H, p, "vec", prior=prior)


# ---- 33 .. 96 rows, dense formats, S a multiple of 256: the kernel whose eight waves share the staged states
# (tuning key 8 = 1 switches back to the kernel whose waves stage their own)
@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("M,K,S,g", [(33, 1024, 512, 128), (48, 4096, 256, 64), (49, 2048, 768, -1), (64, 8192, 256, 128),
                                     (65, 1024, 1024, 64), (96, 4096, 512, 128), (80, 320, 256, 64), (40, 64, 256, 64),
                                     (2, 2048, 256, 128), (16, 1024, 512, 64), (17, 4096, 256, 128), (32, 2048, 512, -1)])
def test_shared_staging_rows(H, bits, M, K, S, g):
    capi = H.capi
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=M + K + S)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    runs = []
    capi.tune(8, 2)                          # whatever the shape (by default: large matrices only)
    try:
        ws = capi.new_matmul_workspace(1, M, K, S, False)
        for _ in range(2):
            o = torch.full((1, M, S), 9.0, dtype=torch.float16, device="cuda")
            capi.matmul(bits, o, d["matrix"], d["states"], d["scales"], d["zeros"], g, None, ws)
            torch.cuda.synchronize()
            runs.append(o.cpu().numpy())
    finally:
        capi.tune(8, 0)
    H.assert_product_close(runs[0], exact, f32, kind="vec")
    assert np.array_equal(runs[0], runs[1])
    capi.tune(8, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        capi.tune(8, 0)
    assert O.max_rel_error(ref.astype(np.float64), runs[0]) < H.TOL_EXACT


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_shared_staging_rows_exponent_mode_and_batches(H, bits):
    H.capi.tune(8, 2)
    try:
        _shared_staging_exponent_and_batches(H, bits)
    finally:
        H.capi.tune(8, 0)


def _shared_staging_exponent_and_batches(H, bits):
    p = _problem(bits, K=2048, S=512, M=1, B=50, group_size=128, seed=21)
    p["scales"][1, 40:48] *= np.float16(-1)
    p["scales"][9, 300] *= np.float16(-1)
    prior = np.random.default_rng(5).standard_normal((50, 1, 512)).astype(np.float16)
    _check(H, p, "vec", prior=prior)                  # the matvec entry adds onto outs
    q = _problem(bits, K=1024, S=256, M=12, B=4, group_size=64, seed=22)
    _check(H, q, "mtx")


@pytest.mark.parametrize("M", [17, 32, 40, 64, 96])
def test_shared_staging_rows_default_rule_large_matrix(H, M):
    """K=4096, S=8192 (32 M weights): every row count from 17 on takes the shared-staging kernel by default"""
    p = _problem(4, K=4096, S=8192, M=M, group_size=128, seed=M)
    _check(H, p, "mtx")


@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("M,K,S,g", [(97, 1024, 512, 128), (128, 4096, 256, 64), (130, 2048, 768, -1), (200, 1024, 1024, 64),
                                     (256, 2048, 512, 128), (129, 320, 256, 64), (257, 1024, 512, 64), (300, 2048, 256, 128),
                                     (384, 512, 768, 64), (449, 1536, 256, -1), (512, 1024, 512, 128)])
def test_shared_staging_up_to_512_rows(H, bits, M, K, S, g):
    """97 ... 512 rows (row blocks of up to 64 or 128 rows): the weights are dequantised with the reference's two
    roundings, so the matmul tolerance against the product on fp16 weights holds"""
    assert "wide_rows_kernel" in H.capi.describe_launch("mtx", bits, 1, M, K, S, g)
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=M + K + S)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((1, M, S), 2.0, np.float16))
    H.assert_product_close(got, exact, f32, kind="mtx")
    H.capi.tune(8, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        H.capi.tune(8, 0)
    assert O.max_rel_error(ref.astype(np.float64), got) < H.TOL_EXACT_MTX


# ---- 16:32 through the shared-staging kernel
@pytest.mark.parametrize("M,K,S,g", [(17, 1024, 512, 64), (33, 2048, 256, 128), (64, 4096, 256, 64), (65, 1024, 1024, -1),
                                     (96, 2048, 512, 64), (128, 4096, 256, 64), (200, 1024, 768, 128), (256, 2048, 512, 64),
                                     (2, 512, 256, 64), (40, 64, 256, 64)])
def test_shared_staging_sparse(H, M, K, S, g):
    capi = H.capi
    p = O.make_problem(bits=4, K=K, S=S, M=M, group_size=g, sparse=True, seed=M + K + S)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    runs = []
    capi.tune(8, 2)                          # whatever the shape
    try:
        ws = capi.new_matmul_workspace(1, M, K, S, True)
        for _ in range(2):
            o = torch.full((1, M, S), 9.0, dtype=torch.float16, device="cuda")
            capi.matmul(4, o, d["matrix"], d["states"], d["scales"], d["zeros"], g, d["mask"], ws)
            torch.cuda.synchronize()
            runs.append(o.cpu().numpy())
    finally:
        capi.tune(8, 0)
    H.assert_product_close(runs[0], exact, f32, kind="mtx")       # (the reference's two roundings per weight)
    assert np.array_equal(runs[0], runs[1])
    capi.tune(8, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        capi.tune(8, 0)
    assert O.max_rel_error(ref.astype(np.float64), runs[0]) < H.TOL_EXACT


def test_shared_staging_sparse_exponent_mode_batches_and_crowded_masks(H):
    H.capi.tune(8, 2)
    try:
        p = O.make_problem(bits=4, K=2048, S=512, M=1, B=50, group_size=64, sparse=True, seed=31)
        p["scales"][1, 40:48] *= np.float16(-1)
        p["scales"][9, 300] *= np.float16(-1)
        prior = np.random.default_rng(5).standard_normal((50, 1, 512)).astype(np.float16)
        _check(H, p, "vec", prior=prior)              # the matvec entry adds onto outs
        # masks whose kept rows crowd one end of a block
        K, S, M = 256, 256, 40
        rng = np.random.default_rng(3)
        codes = rng.integers(0, 16, size=(K, S), dtype=np.uint8)
        keep = np.zeros((K // 32, 32, S), dtype=bool)
        keep[0, :16] = True
        keep[1, 16:] = True
        keep[2, 8:24] = True
        keep[3, ::2] = True
        keep[4, :8] = True
        keep[4, 24:] = True
        keep[5, 1::2] = True
        keep[6, :4] = True
        keep[6, 20:] = True
        keep[7, 3:19] = True
        keep = keep.reshape(K, S)
        matrix, mask = O.sparse_pack(np.ascontiguousarray(codes.T), np.ascontiguousarray(keep.T).astype(np.uint8))
        q = dict(B=1, M=M, S=S, K=K, bits=4, group_size=64, matrix=matrix, sparse_mask=mask, keep=keep,
                 codes=np.where(keep, codes, np.uint8(0)), states=rng.standard_normal((1, M, K)).astype(np.float16),
                 scales=rng.uniform(0.001, 0.02, size=(K // 64, S)).astype(np.float16),
                 zeros=rng.uniform(0, 15, size=(K // 64, S)).astype(np.float16))
        _check(H, q, "mtx")
    finally:
        H.capi.tune(8, 0)


@pytest.mark.parametrize("M", [40, 100, 128])
def test_shared_staging_sparse_default_rule(H, M):
    """K=4096, S=8192 (32 M weights), 16:32: 33 rows and more take the shared-staging kernel by default"""
    p = O.make_problem(bits=4, K=4096, S=8192, M=M, group_size=64, sparse=True, seed=M)
    _check(H, p, "mtx")


# ---- row blocks of 96 / 128 rows (dense formats): one workgroup keeps up to eight 16-row tiles per column pair
# and stages two rows of states per thread.  Taken where K is not split at all or split into long shares.
@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("M,K,S,g", [(100, 512, 512, 64), (128, 512, 256, 128), (70, 320, 768, 64), (65, 448, 256, -1),
                                     (256, 512, 512, 128), (129, 512, 256, 64), (200, 256, 768, 64)])
def test_tall_row_blocks(H, bits, M, K, S, g):
    tiles = H.capi.describe_launch("mtx", bits, 1, M, K, S, g)
    assert "wide_rows_kernel" in tiles and ("row_tiles=6" in tiles or "row_tiles=8" in tiles), tiles
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=M + K + S)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((1, M, S), 2.0, np.float16))
    H.assert_product_close(got, exact, f32, kind="mtx")
    again = H.run_capi(p, d, "mtx")
    assert np.array_equal(got, again)
    H.capi.tune(8, 1)                          # the kernel whose waves stage their own states
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        H.capi.tune(8, 0)
    assert O.max_rel_error(ref.astype(np.float64), got) < H.TOL_EXACT_MTX


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_tall_row_blocks_exponent_mode_and_batches(H, bits):
    """exponent-mode columns take the general decode of the same kernel; batches flatten into rows"""
    p = _problem(bits, K=512, S=512, M=25, B=5, group_size=128, seed=31)
    assert "row_tiles=8" in H.capi.describe_launch("mtx", bits, 5, 25, 512, 512, 128)
    p["scales"][1, 40:48] *= np.float16(-1)
    p["scales"][3, 300] *= np.float16(-1)
    _check(H, p, "mtx")


@pytest.mark.parametrize("bits,M", [(4, 128), (4, 70), (3, 128), (2, 96)])
def test_tall_row_blocks_full_size_split_k(H, bits, M):
    """K=5120, S=20480: 80 strips, K split three ways, partial tiles of 96 / 128 rows handed over"""
    tiles = H.capi.describe_launch("mtx", bits, 1, M, 5120, 20480, 128)
    assert "row_blocks=1 ksplit=3" in tiles and ("row_tiles=6" in tiles or "row_tiles=8" in tiles), tiles
    p = _problem(bits, K=5120, S=20480, M=M, group_size=128, seed=M)
    _check(H, p, "mtx")


@pytest.mark.parametrize("M,K,S,g", [(100, 512, 512, 64), (128, 512, 256, 128), (70, 320, 1024, 64), (96, 448, 256, -1),
                                     (200, 512, 512, 64)])
def test_tall_row_blocks_sparse(H, M, K, S, g):
    """16:32 in row blocks of 96 / 128 rows (two units of weights in flight per wave)"""
    tiles = H.capi.describe_launch("mtx", 4, 1, M, K, S, g, sparse=True)
    assert "wide_rows_kernel<bits=4,16:32" in tiles and ("row_tiles=6" in tiles or "row_tiles=8" in tiles), tiles
    p = O.make_problem(bits=4, K=K, S=S, M=M, group_size=g, sparse=True, seed=M + K + S)
    p["scales"].reshape(-1, S)[-1, 8:12] *= np.float16(-1)            # a few exponent-mode columns
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((1, M, S), 2.0, np.float16))
    H.assert_product_close(got, exact, f32, kind="mtx")
    assert np.array_equal(got, H.run_capi(p, d, "mtx"))
    H.capi.tune(8, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        H.capi.tune(8, 0)
    assert O.max_rel_error(ref.astype(np.float64), got) < H.TOL_EXACT_MTX


def test_tall_row_blocks_sparse_full_size_split_k(H):
    """K=5120, S=20480, g=64, 128 rows: one block of eight tiles, K split three ways"""
    tiles = H.capi.describe_launch("mtx", 4, 1, 128, 5120, 20480, 64, sparse=True)
    assert "wide_rows_kernel<bits=4,16:32,row_tiles=8> strips=80 row_blocks=1 ksplit=3" in tiles, tiles
    p = O.make_problem(bits=4, K=5120, S=20480, M=128, group_size=64, sparse=True, seed=9)
    _check(H, p, "mtx")


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (4, True)])
def test_many_batch_elements_through_the_matvec_entry(H, bits, sparse):
    """300 batch elements of one row each: the matvec entry flattens them into rows of the shared-staging kernel
    and adds onto the prior contents of outs"""
    g = 64 if sparse else 128
    assert "wide_rows_kernel" in H.capi.describe_launch("vec", bits, 300, 1, 1024, 512, g, sparse=sparse)
    kw = {} if bits == 4 else dict(scale_range=(0.004, 0.08), zero_const=3.5)
    p = O.make_problem(bits=bits, K=1024, S=512, M=1, B=300, group_size=g, sparse=sparse, seed=77, **kw)
    prior = np.random.default_rng(8).standard_normal((300, 1, 512)).astype(np.float16)
    _check(H, p, "vec", prior=prior)


# ---- two to four rows through the matvec kernel (a row of states per MFMA result register; dense formats, K <= 5120,
# outputs of 8192 columns and more -- three and four rows: more than 16384)
@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("R", [2, 3, 4])
@pytest.mark.parametrize("K,S,g", [(4096, 22016, 128), (5120, 17408, 64), (4096, 18432, -1)])
def test_two_to_four_rows_equal_the_matvec_row_by_row(H, bits, R, K, S, g):
    """the matmul entry (overwrites outs) and the matvec entry with R batch elements (adds onto outs) give, bit for
    bit, what R calls of the one-row matvec give; exponent-mode columns included"""
    capi = H.capi
    assert "rows=" in capi.describe_launch("mtx", bits, 1, R, K, S, g)
    assert "rows=" in capi.describe_launch("vec", bits, R, 1, K, S, g)
    p = _problem(bits, K=K, S=S, M=R, group_size=g, seed=R + K + S)
    sc, ze = p["scales"].reshape(-1, S), p["zeros"].reshape(-1, S)
    sc[0, 8:12] *= np.float16(-1)
    sc[-1, S - 1] *= np.float16(-1)
    # (exponent-mode weights are fp16(z -+ s 2^e), rounded once per weight by the reference and the oracle, while the
    # matvec adds z sum(x) in fp32: with z near 15 that rounding alone is worth 6e-3 of an output -- a small z keeps
    # the comparison about the kernel)
    ze[0, 8:12] = np.float16(0.25)
    ze[-1, S - 1] = np.float16(0.25)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((1, R, S), 7.0, np.float16))
    H.assert_product_close(got, exact, f32, kind="vec")
    ws = capi.new_matmul_workspace(1, R, K, S, False)
    rows = torch.zeros((1, R, S), dtype=torch.float16, device="cuda")
    for r in range(R):
        capi.matvec(bits, rows[:, r:r + 1], d["matrix"], d["states"][:, r:r + 1].contiguous(), d["scales"], d["zeros"], g, None, ws)
    torch.cuda.synchronize()
    assert np.array_equal(got, rows.cpu().numpy())
    # the matvec entry: R batch elements, prior contents of outs added
    prior = np.random.default_rng(R).standard_normal((R, 1, S)).astype(np.float16)
    outs = torch.from_numpy(prior).cuda()
    want = torch.from_numpy(prior).cuda()
    xb = d["states"].reshape(R, 1, K).contiguous()
    capi.matvec(bits, outs, d["matrix"], xb, d["scales"], d["zeros"], g, None, ws)
    for r in range(R):
        capi.matvec(bits, want[r:r + 1], d["matrix"], xb[r:r + 1], d["scales"], d["zeros"], g, None, ws)
    torch.cuda.synchronize()
    assert np.array_equal(outs.cpu().numpy(), want.cpu().numpy())


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_two_to_four_rows_full_size(H, bits):
    """K=5120, S=20480, three rows: 160 strips, four splits of K handing over three slot rows each"""
    assert "rows=4> strips=160 splits=4" in H.capi.describe_launch("mtx", bits, 1, 3, 5120, 20480, 128)
    p = _problem(bits, K=5120, S=20480, M=3, group_size=128, seed=12)
    _check(H, p, "mtx")
    again = _problem(bits, K=5120, S=20480, M=2, group_size=128, seed=13)       # the slots come back clean
    _check(H, again, "mtx")


def test_two_rows_long_k_with_prefetch(H):
    """K=8192, S=20480, two rows: the two-row kernel with the next unit's loads in flight"""
    tiles = H.capi.describe_launch("mtx", 4, 1, 2, 8192, 20480, 128)
    assert "prefetch=1,rows=2>" in tiles, tiles
    p = _problem(4, K=8192, S=20480, M=2, group_size=128, seed=14)
    _check(H, p, "mtx")


@pytest.mark.parametrize("bits,sparse,K,S,g", [(4, False, 5120, 20480, 128), (3, False, 4096, 6144, 64), (2, False, 2048, 4096, -1),
                                                (4, True, 4096, 8192, 64), (4, False, 128, 128, 128)])
def test_one_row_through_the_matmul_entry(H, bits, sparse, K, S, g):
    """a single row through the matmul entry runs the matvec kernel and overwrites outs: bit for bit the matvec
    entry's result on zeroed outs; a column in exponent mode included.  Without a workspace, where the matvec
    would need one, a tile kernel serves it as before."""
    capi = H.capi
    line = capi.describe_launch("mtx", bits, 1, 1, K, S, g, sparse)
    assert line.startswith("matvec_kernel<"), line
    p = _problem(bits, K=K, S=S, M=1, group_size=g, sparse=sparse, seed=K + bits)
    p["scales"][:, 5] = -p["scales"][:, 5]
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    ws = capi.new_matmul_workspace(1, 1, K, S, sparse)
    args = (d["matrix"], d["states"], d["scales"], d["zeros"], g, d["mask"])
    via_vec = torch.zeros((1, 1, S), dtype=torch.float16, device="cuda")
    capi.matvec(bits, via_vec, *args, ws)
    for _ in range(2):
        via_mtx = torch.full((1, 1, S), -77.0, dtype=torch.float16, device="cuda")
        capi.matmul(bits, via_mtx, *args, ws)
        torch.cuda.synchronize()
        capi.workspace_status(ws)
        assert torch.equal(via_mtx, via_vec)
    H.assert_product_close(via_mtx.cpu().numpy(), exact, f32, kind="vec")
    no_ws = torch.full((1, 1, S), -77.0, dtype=torch.float16, device="cuda")
    capi.matmul(bits, no_ws, *args, None)
    torch.cuda.synchronize()
    H.assert_product_close(no_ws.cpu().numpy(), exact, f32, kind="vec")


@pytest.mark.parametrize("bits", [4, 3])
def test_two_row_blocks_of_32_on_a_narrow_output_long_k(H, bits):
    """49 ... 64 rows against K=11008, S=4096: the shared-staging kernel in two blocks of 32 rows, K split eight ways;
    an exponent-mode group included"""
    M, K, S, g = 60, 11008, 4096, 128
    tiles = H.capi.describe_launch("mtx", bits, 1, M, K, S, g)
    assert tiles.startswith("wide_rows_kernel<bits=%d,dense,row_tiles=2> strips=16 row_blocks=2 ksplit=8" % bits), tiles
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=61)
    p["scales"][40, 1000:1004] *= np.float16(-1)
    p["zeros"][40, 1000:1004] = np.float16(0.5)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx", outs_init=np.full((1, M, S), 2.0, np.float16))
    H.assert_product_close(got, exact, f32, kind="mtx")
    assert np.array_equal(got, H.run_capi(p, d, "mtx"))


@pytest.mark.parametrize("bits,sparse,B", [(4, False, 1100), (3, False, 1025), (4, True, 600)])
def test_more_batch_elements_than_one_launch_takes(H, bits, sparse, B):
    """more than 512 batch elements of one row through the matvec entry: chunks of up to 512 through the few-row kernels
    (1 025: two chunks and the plain matvec for the last row), added onto the prior contents of outs"""
    g = 64 if sparse else 128
    assert "wide_rows_kernel" in H.capi.describe_launch("vec", bits, B, 1, 1024, 512, g, sparse=sparse)
    kw = {} if bits == 4 else dict(scale_range=(0.004, 0.08), zero_const=3.5)
    p = O.make_problem(bits=bits, K=1024, S=512, M=1, B=B, group_size=g, sparse=sparse, seed=B, **kw)
    prior = np.random.default_rng(B).standard_normal((B, 1, 512)).astype(np.float16)
    _check(H, p, "vec", prior=prior)


# ---- more 64-column strips than CUs, up to 16 rows: the work is shared out evenly over one workgroup per CU.
# int4 and 16:32: the workgroups share the strips' units (a strip that two of them share is summed through the
# workspace); int3 and int2 with at most a quarter more strips than CUs: no sharing, a workgroup takes 64 or 80
# columns.  Tuning key 9 = 1: a workgroup per strip.
EVEN_SHAPES = [(8, 3072, 16448, 128), (5, 3072, 20480, 64), (16, 3072, 20416, -1), (9, 3200, 17408, 64),
               (6, 10240, 20544, 128), (2, 4096, 18432, 256)]


def _evenly_shared(line):
    return ("balanced" in line and "workgroups=256" in line) or ("columns_per_lane=4+1" in line and "strips=256" in line)


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (2, False), (4, True)])
@pytest.mark.parametrize("M,K,S,g", EVEN_SHAPES)
def test_few_rows_evenly_shared_launch(H, bits, sparse, M, K, S, g):
    capi = H.capi
    line = capi.describe_launch("mtx", bits, 1, M, K, S, g, sparse)
    if not line.startswith("matvec_kernel"):             # (two to four rows of a dense format may go to the matvec kernel)
        assert _evenly_shared(line), line
        assert ("4+1" in line) == (not sparse and bits != 4 and S <= 20480)
    p = _problem(bits, K=K, S=S, M=M, group_size=g, seed=M + S, sparse=sparse)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    ws = capi.new_matmul_workspace(1, M, K, S, sparse)
    outs = []
    for _ in range(3):                                   # one workspace: the strips' counters must come back to zero
        o = torch.full((1, M, S), -5.0, dtype=torch.float16, device="cuda")
        capi.matmul(bits, o, d["matrix"], d["states"], d["scales"], d["zeros"], g, d["mask"], ws)
        torch.cuda.synchronize()
        outs.append(o.cpu().numpy())
    capi.workspace_status(ws)                            # (raises if a hand-over has failed on it)
    # (one group over all of K: the sums of the offsets reach 10^6 and more in fp32 -- the floor of 1 x RMS only)
    H.assert_product_close(outs[0], exact, f32, kind="vec", tight=g > 0 and line.startswith(("skinny_kernel", "matvec_kernel")))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    capi.tune(9, 1)                                      # a workgroup per strip
    try:
        assert not _evenly_shared(capi.describe_launch("mtx", bits, 1, M, K, S, g, sparse))
        ref = H.run_capi(p, d, "mtx")
    finally:
        capi.tune(9, 0)
    assert O.max_rel_error(ref.astype(np.float64), outs[0]) < H.TOL_EXACT


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (2, False), (4, True)])
def test_few_rows_evenly_shared_exponent_mode_batches_and_prior_outs(H, bits, sparse):
    # five batch elements through the matvec entry, which adds onto outs; exponent-mode columns in a strip that two
    # workgroups share (strip 1 of 320: workgroup 0 takes its first quarter) and in one that a workgroup has to itself
    K, S, g = 3072, 20480, 128 if not sparse else 64
    assert _evenly_shared(H.capi.describe_launch("vec", bits, 5, 1, K, S, g, sparse))
    p = _problem(bits, K=K, S=S, M=1, B=5, group_size=g, seed=12, sparse=sparse)
    p["scales"][0, 64 + 5] *= np.float16(-1)
    p["scales"][(K // g) - 1, 64 + 40:64 + 44] *= np.float16(-1)
    p["scales"][3, 4 * 64 + 17] *= np.float16(-1)
    prior = np.random.default_rng(2).standard_normal((5, 1, S)).astype(np.float16)
    _check(H, p, "vec", prior=prior)


def test_few_rows_shared_strips_take_turns_on_one_workspace(H):
    """a matvec, the few-row product with shared strips and a matvec again on one workspace: the strips' counters and
    partial tiles must not disturb the matvec's hand-over slots, nor the other way round"""
    capi = H.capi
    K, S, g = 3072, 20480, 128
    assert "balanced" in capi.describe_launch("mtx", 4, 1, 8, K, S, g)
    pv = _problem(4, K=K, S=S, M=1, group_size=g, seed=3)
    pm = dict(pv, M=8, states=np.random.default_rng(4).standard_normal((1, 8, K)).astype(np.float16))
    dv, dm = H.dev_problem(pv), H.dev_problem(pm)
    ws = capi.new_matmul_workspace(1, 8, K, S, False)
    assert ws.numel() * ws.element_size() >= capi.lib().int4mm_workspace_bytes(S)
    ev, fv = H.oracles(pv)
    em, fm = H.oracles(pm)
    for _ in range(2):
        ov = torch.zeros((1, 1, S), dtype=torch.float16, device="cuda")
        capi.matvec(4, ov, dv["matrix"], dv["states"], dv["scales"], dv["zeros"], g, None, ws)
        om = torch.zeros((1, 8, S), dtype=torch.float16, device="cuda")
        capi.matmul(4, om, dm["matrix"], dm["states"], dm["scales"], dm["zeros"], g, None, ws)
        torch.cuda.synchronize()
        H.assert_product_close(ov.cpu().numpy(), ev, fv, kind="vec")
        H.assert_product_close(om.cpu().numpy(), em, fm, kind="vec")
    capi.workspace_status(ws)
