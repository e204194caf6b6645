"""Split-K of the pipelined matmul: shapes with few output tiles run several
workgroups per tile, each over a part of K, and the last one to finish adds the
fp32 partial tiles up.  Checked against the oracle, against the unsplit kernel
(tuning key 6 = 1), on repeated calls through one workspace (the per-tile
counters must come back to zero), with too small a workspace (falls back to the
unsplit kernel) and through the extension, which sizes its own workspace."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402


@pytest.fixture(scope="module")
def H():
    from tests import helpers
    helpers.capi.tune(8, 1)          # (up to 512 rows would otherwise take the few-row path: not the subject here)
    yield helpers
    helpers.capi.tune(8, 0)


def _problem(bits, sparse, **kw):
    if bits != 4:
        kw.setdefault("scale_range", (0.004, 0.08))
        kw.setdefault("zero_const", 3.5 if bits == 3 else 1.5)
    return O.make_problem(bits=bits, sparse=sparse, **kw)


FORMATS = [(4, False), (3, False), (2, False), (4, True)]


@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("M,K,S,g,B", [(256, 2048, 512, 128, 1), (200, 1536, 256, 64, 1), (512, 4096, 256, -1, 1),
                                       (256, 1024, 256, 64, 3), (400, 2560, 768, 128, 1)])
def test_split_k_matches_oracle_and_unsplit(H, bits, sparse, M, K, S, g, B):
    capi = H.capi
    p = _problem(bits, sparse, K=K, S=S, M=M, group_size=g, seed=M + K, B=B)
    assert capi.matmul_workspace_bytes(B, M, K, S, sparse) > capi.lib().int4mm_workspace_bytes(S), "shape should split"
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    got = H.run_capi(p, d, "mtx")
    H.assert_product_close(got, exact, f32, kind="mtx")
    capi.tune(6, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        capi.tune(6, 0)
    assert O.max_rel_error(ref.astype(np.float64), got) < H.TOL_EXACT


@pytest.mark.parametrize("bits,sparse", [(4, False), (4, True)])
def test_split_k_repeated_calls_share_a_workspace(H, bits, sparse):
    capi = H.capi
    p = _problem(bits, sparse, K=2048, S=512, M=256, group_size=128, seed=5)
    d = H.dev_problem(p)
    ws = capi.new_matmul_workspace(1, 256, 2048, 512, sparse)
    outs = torch.zeros((1, 256, 512), dtype=torch.float16, device="cuda")
    results = []
    for _ in range(4):
        outs.fill_(7.0)
        capi.matmul(bits, outs, d["matrix"], d["states"], d["scales"], d["zeros"], 128, d["mask"], ws)
        torch.cuda.synchronize()
        results.append(outs.cpu().numpy().copy())
    for r in results[1:]:
        assert np.array_equal(r, results[0])              # the sum has one order whoever arrives last
    exact, f32 = H.oracles(p)
    H.assert_product_close(results[0], exact, f32, kind="mtx")
    kept_zero = (ws.numel() // 2) & ~4095
    assert int(ws[:kept_zero].to(torch.int32).sum()) == 0         # counters and slots are back to zero
    assert int(ws[kept_zero:].to(torch.int32).sum()) != 0         # (the partial tiles were there)


def test_one_workspace_shared_by_calls_of_different_shapes(H):
    """The layout of a workspace depends on its size alone: split matmuls, split few-row products
    and matvecs of different widths may take turns on one buffer."""
    capi = H.capi
    shapes = [("mtx", 4, False, 256, 2048, 512, 128), ("vec", 4, False, 1, 4096, 1024, 128),
              ("mtx", 4, False, 8, 16384, 256, 128), ("vec", 4, True, 1, 2048, 2048, 64),
              ("mtx", 4, True, 256, 2048, 256, 64), ("mtx", 3, False, 40, 8192, 128, 64),
              ("vec", 2, False, 1, 8192, 192, 128), ("mtx", 4, False, 200, 1536, 768, 64)]
    need = max(capi.matmul_workspace_bytes(1, M, K, S, sparse) for _, _, sparse, M, K, S, _ in shapes)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    cases = []
    for kind, bits, sparse, M, K, S, g in shapes:
        p = _problem(bits, sparse, K=K, S=S, M=M, group_size=g, seed=K + S)
        cases.append((kind, bits, g, p, H.dev_problem(p), H.oracles(p)))
    for _ in range(2):
        for kind, bits, g, p, d, (exact, f32) in cases:
            outs = torch.zeros((1, p["M"], p["S"]), dtype=torch.float16, device="cuda")
            fn = capi.matmul if kind == "mtx" else capi.matvec
            fn(bits, outs, d["matrix"], d["states"], d["scales"], d["zeros"], g, d["mask"], ws)
            torch.cuda.synchronize()
            H.assert_product_close(outs.cpu().numpy(), exact, f32, kind="vec" if p["M"] <= 96 else "mtx")


def test_split_k_needs_room_in_the_workspace(H):
    capi = H.capi
    p = _problem(4, False, K=2048, S=512, M=256, group_size=128, seed=6)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    for ws in (None, capi.new_workspace(512)):            # no room for partial tiles: the unsplit kernel runs
        outs = torch.zeros((1, 256, 512), dtype=torch.float16, device="cuda")
        capi.matmul(4, outs, d["matrix"], d["states"], d["scales"], d["zeros"], 128, None, ws)
        torch.cuda.synchronize()
        H.assert_product_close(outs.cpu().numpy(), exact, f32, kind="mtx")


@pytest.mark.parametrize("bits,sparse", [(4, False), (4, True)])
def test_split_k_exponent_mode_columns(H, bits, sparse):
    p = _problem(bits, sparse, K=2048, S=512, M=256, group_size=128, seed=8)
    p["scales"][3, 40:48] *= np.float16(-1)
    p["scales"][9, 300] *= np.float16(-1)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    H.assert_product_close(H.run_capi(p, d, "mtx"), exact, f32, kind="mtx")


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (4, True)])
def test_split_k_through_the_extension(H, bits, sparse):
    p = _problem(bits, sparse, K=2048, S=512, M=256, group_size=128, seed=9)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    for _ in range(2):
        H.assert_product_close(H.run_ext(p, d), exact, f32, kind="mtx")


def test_extension_workspace_survives_changing_shapes(H):
    """The extension keeps one workspace per stream and lets it grow: products of different widths, split or
    not, follow each other through `quant_matmul`."""
    shapes = [(4, False, 16, 8192, 1024, 128), (4, False, 32, 16384, 256, 128), (4, False, 64, 8192, 512, 128),
              (4, True, 8, 8192, 1024, 64), (4, False, 1, 4096, 2048, 128), (4, False, 256, 2048, 512, 128),
              (3, False, 1, 4096, 512, 128), (4, False, 16, 8192, 1024, 128)]
    cases = []
    for bits, sparse, M, K, S, g in shapes:
        p = _problem(bits, sparse, K=K, S=S, M=M, group_size=g, seed=K + S + M)
        cases.append((p, H.dev_problem(p), H.oracles(p)))
    for _ in range(2):
        for p, d, (exact, f32) in cases:
            got = H.run_ext(p, d)
            H.assert_product_close(got, exact, f32, kind="vec" if p["M"] <= 96 else "mtx")


# ---- grids of 256 x 256 tiles whose last round of 256 fills at most half of the GPU: only the tiles of
# that round are split along K (tuning key 7 = 1 switches it off)
@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("M,K,S,g", [(512, 2048, 33280, 128),        # 260 tiles: 4 split in two (shares of 32 K steps)
                                     (2200, 4096, 7424, 64)])        # 261 tiles: 5 split in four
def test_tail_split_matches_oracle_and_unsplit(H, bits, sparse, M, K, S, g):
    capi = H.capi
    p = _problem(bits, sparse, K=K, S=S, M=M, group_size=g, seed=M + K + 1)
    capi.tune(7, 1)
    try:
        plain_bytes = capi.matmul_workspace_bytes(1, M, K, S, sparse)
    finally:
        capi.tune(7, 0)
    assert capi.matmul_workspace_bytes(1, M, K, S, sparse) > plain_bytes, "shape should split its last round"
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    ws = capi.new_matmul_workspace(1, M, K, S, sparse)
    runs = []
    for _ in range(3):                                    # one workspace: the counters come back to zero
        outs = torch.full((1, M, S), 3.0, dtype=torch.float16, device="cuda")
        capi.matmul(bits, outs, d["matrix"], d["states"], d["scales"], d["zeros"], g, d["mask"], ws)
        torch.cuda.synchronize()
        runs.append(outs.cpu().numpy())
    H.assert_product_close(runs[0], exact, f32, kind="mtx")
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
    capi.tune(7, 1)
    try:
        ref = H.run_capi(p, d, "mtx")
    finally:
        capi.tune(7, 0)
    assert O.max_rel_error(ref.astype(np.float64), runs[0]) < H.TOL_EXACT
    # the tiles that were not split are bit-identical to the plain run's
    assert np.array_equal(ref[:, :256, :256], runs[0][:, :256, :256])


def test_sparse_odd_tile_rows_take_split_large_tiles_on_a_long_k(H):
    """16:32, 896 rows (seven tile rows of 128) against K=4096, S=8192: 128 padded 256-row tiles split in two along K
    instead of 224 tiles of 128 rows; without a workspace for the partial tiles the 128-row tiles as before"""
    capi = H.capi
    M, K, S = 896, 4096, 8192
    assert "tile=256x256,plain> tiles=128 ksplit=2" in capi.describe_launch("mtx", 4, 1, M, K, S, 64, True)
    assert "tile=128x256" in capi.describe_launch("mtx", 4, 1, M, K, S, 64, True, workspace_bytes=0)
    assert "tile=128x256" in capi.describe_launch("mtx", 4, 1, M, 2048, S, 64, True)
    p = _problem(4, True, K=K, S=S, M=M, group_size=64, seed=17)
    p["scales"][7, 100:104] *= np.float16(-1)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    junk = np.full((1, M, S), 9.0, np.float16)
    for _ in range(2):
        H.assert_product_close(H.run_capi(p, d, "mtx", outs_init=junk), exact, f32, kind="mtx")
