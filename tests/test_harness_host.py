"""The harness's expected values (plain torch arithmetic on the unpacked codes) against the oracle's decode, on the
CPU: linear and exponent-mode groups, every bit width, with and without a 16:32 mask."""
import numpy as np
import pytest
import torch

from oracle import oracle as O


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (2, False), (4, True)])
def test_reference_matrices_follow_the_oracle_decode(bits, sparse, monkeypatch):
    from int4matmul_kernels_amd import harness
    monkeypatch.setattr(harness, "DEV", "cpu")
    K, S, g = 256, 24, 64
    gen = torch.Generator().manual_seed(bits)
    codes = torch.randint(0, 1 << bits, (K, S), generator=gen, dtype=torch.int32).to(torch.uint8)
    scales = (torch.rand((K // g, S), generator=gen) * 0.07 + 0.004).half()
    scales[1] *= -1                                   # a whole group in exponent mode
    scales[3, ::5] *= -1                              # and single columns of another
    zeros = (torch.rand((K // g, S), generator=gen) * ((1 << bits) - 1)).half()
    keep = None
    if sparse:
        keys = torch.rand((K // 32, 32, S), generator=gen)
        keep = torch.zeros((K // 32, 32, S), dtype=torch.uint8)
        keep.scatter_(1, keys.argsort(dim=1)[:, :16], 1)
        keep = keep.reshape(K, S)
    w16, w32 = harness.reference_matrices(dict(bits=bits, K=K, group=g, codes=codes, scales=scales, zeros=zeros, keep=keep))
    rows = np.arange(K) // g
    want = O.dequant_dynamic(bits, codes.numpy(), scales.numpy()[rows], zeros.numpy()[rows])
    if sparse:
        want = np.where(keep.numpy().astype(bool), want, np.float16(0))
    # (value for value; a dropped row's weight is +0 in the oracle and, as a product with 0, -0 here for a negative weight)
    assert np.array_equal(w16.numpy(), want) and not np.any(np.isnan(want.astype(np.float32)))
    assert np.allclose(w32.numpy(), want.astype(np.float32), rtol=2e-3, atol=1e-6)
