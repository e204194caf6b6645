"""The accuracy / timing harness runs its small configurations through the
`int4matmul` extension and every case passes the reference's 10 % gate
(kernel_test.py:344-348)."""
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
