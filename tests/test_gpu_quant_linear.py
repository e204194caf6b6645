"""QuantLinear: the caller-side holder of the packed formats (quantise / pack on
the device, forward through the `int4matmul` extension)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits,sparse,tol", [(4, False, 0.08), (3, False, 0.17), (2, False, 0.4), (4, True, 0.08)])
@pytest.mark.parametrize("shape", [(1, 1), (2, 5), (1, 300)])
def test_quantise_pack_forward(bits, sparse, tol, shape):
    from int4matmul_kernels_amd.quant_linear import QuantLinear

    torch.manual_seed(bits)
    K, S = 512, 384
    w = (torch.randn((K, S), device="cuda") * 0.05).half()
    keep = None
    if sparse:
        keys = torch.rand((S, K // 32, 32), device="cuda")
        keep = torch.zeros((S, K // 32, 32), dtype=torch.bool, device="cuda")
        keep.scatter_(2, keys.argsort(dim=2)[:, :, :16], True)
        keep = keep.reshape(S, K).t().contiguous()
    bias = torch.randn((S,), device="cuda").half()
    layer = QuantLinear.from_float(w, bits=bits, group_size=64, keep=keep, bias=bias)
    wq = layer.dequantized_weight()
    target = w if keep is None else w * keep
    # quantisation error of round-to-nearest: at most half a step of the group's range
    step = (w.float().reshape(K // 64, 64, S).amax(1) - w.float().reshape(K // 64, 64, S).amin(1)) / ((1 << bits) - 1)
    err = (wq.float() - target.float()).abs().reshape(K // 64, 64, S).amax(1)
    assert torch.all(err <= 0.51 * step + 2e-3)
    if keep is not None:
        assert torch.all(wq[~keep] == 0)
    x = torch.randn((*shape, K), device="cuda").half()
    y = layer(x)
    ref = x.float() @ wq.float() + bias.float()
    assert y.shape == (*shape, S) and y.dtype == torch.float16
    rms = ref.pow(2).mean().sqrt()
    assert ((y.float() - ref).abs().max() / rms).item() < 1e-2
    # and close to the unquantised layer within the format's resolution
    full = x.float() @ target.float() + bias.float()
    assert ((y.float() - full).pow(2).mean().sqrt() / full.pow(2).mean().sqrt()).item() < tol


def test_from_packed_round_trip_and_state_dict():
    from int4matmul_kernels_amd.quant_linear import QuantLinear

    w = (torch.randn((256, 128), device="cuda") * 0.1).half()
    a = QuantLinear.from_float(w, bits=4, group_size=-1)
    b = QuantLinear.from_packed(4, a.matrix, a.scales, a.zeros, -1)
    c = QuantLinear(4, 256, 128, group_size=-1)
    c.load_state_dict(a.state_dict())
    x = torch.randn((3, 1, 256), device="cuda").half()
    assert torch.equal(a(x), b(x)) and torch.equal(a(x), c(x))
    with pytest.raises(ValueError):
        QuantLinear(3, 256, 128, sparse=True)
