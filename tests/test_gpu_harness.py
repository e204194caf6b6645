"""The accuracy / timing harness runs through the `int4matmul` extension and every
case passes the reference's 10 % gate (kernel_test.py:344-348): its small
configurations, and one full-size benchmark configuration per format."""
import pytest

pytestmark = pytest.mark.gpu


def test_harness_quick_configurations():
    from int4matmul_kernels_amd import harness

    rows = harness.main(["--quick", "--repeats", "3"])
    assert len(rows) == len(harness.QUICK)
    for r in rows:
        assert r["ok"], r
        assert r["err_quant"] < 0.1
        assert r["quant_event_us"] > 0


def test_harness_full_size_row_per_format():
    from int4matmul_kernels_amd import harness

    names = ["C2", "C3", "C4v", "C5m3", "C5v2"]
    rows = harness.main(["--only", ",".join(names), "--repeats", "2"])
    assert [r["name"] for r in rows] == names
    for r in rows:
        assert r["ok"] and r["err_quant"] < 1e-2, r            # (mean relative error; the gate itself is 0.1)


def test_harness_with_exponent_mode_groups():
    """every second group of every column in exponent mode: the harness's own truth (from the unpacked codes, in
    plain torch arithmetic) holds every format's kernels to the same gate"""
    from int4matmul_kernels_amd import harness

    rows = harness.main(["--quick", "--repeats", "2", "--exponent-every", "2"])
    assert len(rows) == len(harness.QUICK)
    for r in rows:
        assert r["ok"] and r["err_quant"] < 1e-2, r
