"""Failure handling of the matvec's cross-workgroup hand-over, forced from the host:
with the bounded wait cut down to a single poll the reader gives up on slots that
are not there yet.  Such a run must never return a silently wrong number: the
outputs it could not finish are NaN, the workspace is marked, later calls on it
return NaN and report INT4MM_ERR_HANDOVER until it has been zero-filled again.
Every kernel still runs to its normal end (the wait is bounded by construction)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def test_timed_out_hand_over_poisons_instead_of_lying():
    from tests import helpers as H
    capi = H.capi
    p = O.make_problem(K=5120, S=20480, M=1, bits=4, group_size=128, seed=3)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    ws = capi.new_workspace(p["S"])

    def run():
        outs = torch.zeros((1, 1, p["S"]), dtype=torch.float16, device="cuda")
        capi.matvec(4, outs, d["matrix"], d["states"], d["scales"], d["zeros"], 128, None, ws)
        torch.cuda.synchronize()
        return outs.cpu().numpy()

    H.assert_product_close(run(), exact, f32)
    capi.workspace_status(ws)                                # healthy
    capi.tune(10, 1)                                         # one poll, then give up
    try:
        timed_out = False
        for _ in range(20):
            got = run()
            try:
                capi.workspace_status(ws)
            except capi.Int4mmError as e:
                assert e.code == 9
                timed_out = True
                break
            H.assert_product_close(got, exact, f32)          # no time-out: the result is simply right
    finally:
        capi.tune(10, 0)
    if not timed_out:
        pytest.skip("every slot was there at the first poll in 20 runs: nothing timed out")
    bad = np.isnan(got.astype(np.float32))
    assert bad.any()
    ok = ~bad
    # what was finished is right, what was not is NaN -- nothing in between
    assert O.max_rel_error(f32[ok], got[ok]) < H.TOL_F32
    again = run()                                            # default wait again, same workspace: poisoned
    assert np.isnan(again.astype(np.float32)).all()
    with pytest.raises(capi.Int4mmError):
        capi.workspace_status(ws)
    ws.zero_()                                               # (what int4mm_workspace_init does)
    H.assert_product_close(run(), exact, f32)
    capi.workspace_status(ws)


def test_timed_out_hand_over_with_three_rows():
    """the same for three rows of states through the matvec kernel (a slot row per split and row)"""
    from tests import helpers as H
    capi = H.capi
    K, S, R = 5120, 20480, 3
    assert "rows=" in capi.describe_launch("mtx", 4, 1, R, K, S, 128)
    p = O.make_problem(K=K, S=S, M=R, bits=4, group_size=128, seed=4)
    d = H.dev_problem(p)
    exact, f32 = H.oracles(p)
    ws = capi.new_matmul_workspace(1, R, K, S, False)

    def run():
        outs = torch.full((1, R, S), 3.0, dtype=torch.float16, device="cuda")
        capi.matmul(4, outs, d["matrix"], d["states"], d["scales"], d["zeros"], 128, None, ws)
        torch.cuda.synchronize()
        return outs.cpu().numpy()

    H.assert_product_close(run(), exact, f32)
    capi.workspace_status(ws)
    capi.tune(10, 1)
    try:
        timed_out = False
        for _ in range(20):
            got = run()
            try:
                capi.workspace_status(ws)
            except capi.Int4mmError as e:
                assert e.code == 9
                timed_out = True
                break
            H.assert_product_close(got, exact, f32)
    finally:
        capi.tune(10, 0)
    if not timed_out:
        pytest.skip("every slot was there at the first poll in 20 runs: nothing timed out")
    bad = np.isnan(got.astype(np.float32))
    assert bad.any()
    ok = ~bad
    assert O.max_rel_error(f32[ok], got[ok]) < H.TOL_F32
    assert np.isnan(run().astype(np.float32)).all()          # poisoned until zero-filled
    ws.zero_()
    H.assert_product_close(run(), exact, f32)
    capi.workspace_status(ws)
