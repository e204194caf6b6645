"""int4mm_matvec_static -- the matvec entry point that allocates nothing -- against
int4mm_matvec, through the C ABI: two calls in a row on the library's built-in
scratch array, the second with a smaller input, both bit for bit equal to the
entry point that takes a caller's workspace (same kernels, deterministic
summation order), and no device allocation in between."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    import helpers
    return helpers


def _both(H, p, d, prior):
    capi = H.capi
    S = p["S"]
    want = H.t(prior).clone()
    ws = capi.new_workspace(S)
    capi.matvec(p["bits"], want, d["matrix"], d["states"], d["scales"], d["zeros"], p["group_size"], d["mask"], ws)
    got = H.t(prior).clone()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    capi.matvec_static(p["bits"], got, d["matrix"], d["states"], d["scales"], d["zeros"], p["group_size"], d["mask"])
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before      # (torch's allocator saw nothing)
    return want.cpu().numpy(), got.cpu().numpy()


def test_static_scratch_matvec_matches_workspace_matvec(H):
    # first call: K split over several workgroups per strip (the hand-over slots are in use);
    # second call: a smaller matrix on the same scratch, which must have been left clean
    shapes = [dict(K=5120, S=20480, bits=4, group_size=128, sparse=False),
              dict(K=2048, S=4096, bits=4, group_size=64, sparse=False),
              dict(K=4096, S=2048, bits=4, group_size=64, sparse=True),
              dict(K=1024, S=512, bits=3, group_size=128, sparse=False)]
    for i, sh in enumerate(shapes):
        p = O.make_problem(M=1, seed=40 + i, **sh)
        d = H.dev_problem(p)
        rng = np.random.default_rng(i)
        prior = rng.standard_normal((1, 1, p["S"])).astype(np.float16)       # the matvec adds onto outs
        want, got = _both(H, p, d, prior)
        assert np.array_equal(want.view(np.uint16), got.view(np.uint16)), f"shape {i} differs"
        exact, f32 = H.oracles(p)
        H.assert_product_close(got, exact, f32, prior=prior, kind="vec")


def test_static_scratch_batch_and_limit(H):
    capi = H.capi
    # a batch of rows takes the few-row kernel, whose split-K partials also live in the scratch
    p = O.make_problem(K=8192, S=1024, M=1, B=4, bits=4, group_size=128, seed=50)
    d = H.dev_problem(p)
    prior = np.zeros((4, 1, 1024), np.float16)
    want, got = _both(H, p, d, prior)
    assert np.array_equal(want.view(np.uint16), got.view(np.uint16))
    # wider than the built-in scratch covers: a clear error, nothing launched
    S = 32768 + 64
    outs = torch.zeros((1, 1, S), dtype=torch.float16, device="cuda")
    m = torch.zeros((8, S), dtype=torch.int32, device="cuda")
    x = torch.zeros((1, 1, 64), dtype=torch.float16, device="cuda")
    sz = torch.zeros((1, S), dtype=torch.float16, device="cuda")
    with pytest.raises(capi.Int4mmError) as e:
        capi.matvec_static(4, outs, m, x, sz, sz, 64, None)
    assert e.value.code == 6
