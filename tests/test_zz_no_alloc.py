"""int4mm_matvec_static -- the matvec entry point that allocates nothing -- against
int4mm_matvec, through the C ABI: two calls in a row on the library's built-in
scratch array, the second with a smaller input, both bit for bit equal to the
entry point that takes a caller's workspace (same kernels, deterministic
summation order), and no device allocation in between; a batch whose launch plan
differs between the two scratch sizes; and the health query / reset of the
built-in array."""
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
    # a first call, so that the module is loaded and the array's address looked up; then the one that is watched
    capi.matvec_static(p["bits"], got, d["matrix"], d["states"], d["scales"], d["zeros"], p["group_size"], d["mask"])
    got.copy_(H.t(prior))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]              # hipMemGetInfo: sees any hipMalloc / hipFree, whoever calls it
    capi.matvec_static(p["bits"], got, d["matrix"], d["states"], d["scales"], d["zeros"], p["group_size"], d["mask"])
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before      # the device's free memory did not move
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


def test_static_scratch_batch_with_another_split_plan(H):
    """64 batch entries at K=8192, S=1024: the few-row kernel's partial sums (512 KiB) fit the built-in
    array's scratch half but not a workspace of int4mm_workspace_bytes(1024), so the two entry points
    take different plans (split / unsplit K): another summation order, the same accuracy class -- both
    are checked against the oracle, not against each other."""
    capi = H.capi
    p = O.make_problem(K=8192, S=1024, M=1, B=64, bits=4, group_size=128, seed=51)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    prior = np.zeros((64, 1, 1024), np.float16)
    ws = capi.new_workspace(1024)
    want = H.t(prior).clone()
    capi.matvec(4, want, d["matrix"], d["states"], d["scales"], d["zeros"], 128, None, ws)
    got = H.t(prior).clone()
    capi.matvec_static(4, got, d["matrix"], d["states"], d["scales"], d["zeros"], 128, None)
    torch.cuda.synchronize()
    kind = H.matmul_kind(dict(p, B=1, M=64))
    H.assert_product_close(want.cpu().numpy(), exact, f32, kind=kind)
    H.assert_product_close(got.cpu().numpy(), exact, f32, kind=kind)


def test_static_scratch_reports_and_clears_a_timed_out_hand_over(H):
    """the failure path of the hand-over on the built-in array: forced from the host (one poll, then give up),
    it poisons the array; the health query with a NULL workspace reports it, the reset with a NULL workspace
    (a fill kernel on the stream, no allocation) clears it"""
    capi = H.capi
    p = O.make_problem(K=5120, S=20480, M=1, bits=4, group_size=128, seed=52)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)

    def run():
        outs = torch.zeros((1, 1, p["S"]), dtype=torch.float16, device="cuda")
        capi.matvec_static(4, outs, d["matrix"], d["states"], d["scales"], d["zeros"], 128, None)
        torch.cuda.synchronize()
        return outs.cpu().numpy()

    H.assert_product_close(run(), exact, f32)
    capi.workspace_status(None)                              # healthy
    capi.workspace_init(None)                                # (a first launch of the fill kernel loads its code object)
    torch.cuda.synchronize()
    capi.tune(10, 1)
    try:
        timed_out = False
        for _ in range(20):
            got = run()
            try:
                capi.workspace_status(None)
            except capi.Int4mmError as e:
                assert e.code == 9
                timed_out = True
                break
            H.assert_product_close(got, exact, f32)
    finally:
        capi.tune(10, 0)
    try:
        if not timed_out:
            pytest.skip("every slot was there at the first poll in 20 runs: nothing timed out")
        assert np.isnan(got.astype(np.float32)).any()
        assert np.isnan(run().astype(np.float32)).all()      # poisoned until it is reset
    finally:
        free_before = torch.cuda.mem_get_info()[0]
        capi.workspace_init(None)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
    capi.workspace_status(None)
    H.assert_product_close(run(), exact, f32)
