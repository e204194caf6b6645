"""Every number of rows from 1 to 520, and the edges of the tile kernels' row paddings beyond, on
full-size matrices.  Which kernel serves a product is decided at launch time from (rows, K, S, format):
the matvec kernel and its two- / four-row forms, the few-row kernels with their row blocks of 16 … 128,
padded and split tiles, whole tiles.  A sweep over the row count crosses every one of those borders at
the shapes the library is measured on; each count is checked against the float64 product on the
oracle's fp16 weights (a library fp64 GEMM on the GPU, from the matrix the CPU oracle decoded), to the
same bars as the other product tests; the outputs start as NaN (the matmul entry overwrites them, with one
row as with many), and the rows behind the last one must stay untouched."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

BEYOND = (576, 640, 641, 767, 768, 769, 1000, 1024, 1025, 1152, 1153, 1535, 1536, 2047)
GUARD_ROWS = 4


def _rel_error(truth, got, floor_frac):
    """oracle.max_rel_error on the GPU: max |got - truth| / max(|truth|, floor_frac * rms(truth))"""
    rms = truth.pow(2).mean().sqrt()
    den = torch.maximum(truth.abs(), floor_frac * rms)
    return ((got.double() - truth).abs() / den).max().item()


@pytest.mark.parametrize("bits,K,S,g,sparse", [
    (4, 5120, 20480, 128, False),
    (4, 5120, 20480, 64, True),
    (4, 8192, 8192, 128, False),
    (3, 4096, 11008, 128, False),
    (2, 20480, 5120, -1, False),
])
def test_every_row_count(bits, K, S, g, sparse):
    from tests import helpers as H
    capi = H.capi
    rows_max = max(BEYOND)
    p = O.make_problem(K=K, S=S, M=rows_max, bits=bits, group_size=g, sparse=sparse, seed=bits * 1000 + K % 997)
    w16 = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], g, p["sparse_mask"])
    d = H.dev_problem(p)
    states = d["states"].reshape(rows_max, K)
    truth = states.double() @ torch.from_numpy(w16).to("cuda").double()       # [rows_max, S]
    sentinel = torch.tensor(float("nan"), dtype=torch.float16)
    buf = torch.empty(((rows_max + GUARD_ROWS) * S,), dtype=torch.float16, device="cuda")
    kernels = set()
    worst = {"vec": 0.0, "mtx": 0.0}
    for M in list(range(1, 521)) + list(BEYOND):
        line = capi.describe_launch("mtx", bits, 1, M, K, S, g, sparse)
        kernels.add(line.split(">")[0])
        kind = "vec" if line.startswith(("skinny_kernel", "matvec_kernel")) else "mtx"
        buf.fill_(sentinel.item())
        outs = buf[:M * S].view(1, M, S)
        x = states[:M].reshape(1, M, K).contiguous()
        ws = capi.new_matmul_workspace(1, M, K, S, sparse)
        capi.matmul(bits, outs, d["matrix"], x, d["scales"], d["zeros"], g, d["mask"], ws)
        torch.cuda.synchronize()
        capi.workspace_status(ws)
        assert torch.isfinite(outs).all(), f"rows={M}: {line}"
        assert torch.isnan(buf[M * S:(M + GUARD_ROWS) * S]).all(), f"rows={M} wrote behind its last row: {line}"
        e = _rel_error(truth[:M], outs[0], 1.0 if kind == "vec" else H.FLOOR_EXACT_MTX)
        assert e < (H.TOL_EXACT if kind == "vec" else H.TOL_EXACT_MTX), f"rows={M}: {e}: {line}"
        worst[kind] = max(worst[kind], e)
    print(f"bits={bits} K={K} S={S} sparse={sparse}: {len(kernels)} kernel forms, worst error {worst}")
    assert len(kernels) >= 4                                 # the sweep did cross the borders
