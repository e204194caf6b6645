"""Bit-exact evidence for the decoders the products really use.

With the identity as states (M = K rows, one 1.0 per row) a product that
dequantises its weights returns them unchanged: the fp32 sum of 1 * w and zeros is
w, and rounding it to fp16 gives back the fp16 weight.  So ``outs`` must equal the
oracle's dequantised matrix (oracle.dequantize_matrix, the restatement of
matmul.cuh:115-136,246-428) BIT FOR BIT -- for every tile kernel variant, the
few-row kernel that dequantises (17 .. 512 rows), with and without split-K, all four
formats, linear and exponent-mode groups.  (Zero weights are compared by value: a
sum of +0.0 and -0.0 is +0.0.)  The matvec and the 2 .. 16 row kernel apply scale
and zero per group in fp32 instead of dequantising, so they are not subject to
this test; they are held to the product tolerances elsewhere.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

FORMATS = [(4, False), (3, False), (2, False), (4, True)]


@pytest.fixture(scope="module")
def H():
    from tests import helpers
    return helpers


def _problem(bits, sparse, K, S, g, seed, expo=True):
    kw = {}
    if bits != 4:
        kw = dict(scale_range=(0.004, 0.08), zero_const=3.5 if bits == 3 else 1.5)
    p = O.make_problem(K=K, S=S, M=K, bits=bits, group_size=g, sparse=sparse, seed=seed, **kw)
    sc = p["scales"]
    if expo:
        sc[1, 3::7] *= np.float16(-1)            # exponent quantisation in some columns of one group
        sc[:, 64:72] *= np.float16(-1)           # and in a few columns throughout
    if bits == 4 and not sparse:
        p["zeros"][0, :16] = np.float16(7.0)     # integer zero: some weights are exactly 0
    p["states"] = np.eye(K, dtype=np.float16)[None]
    return p


def _assert_same_bits(got, want, what):
    got = np.ascontiguousarray(got)
    zero = want == 0
    assert np.array_equal(got[zero] == 0, np.ones(int(zero.sum()), bool)), f"{what}: zero weights"
    a, b = got.view(np.uint16)[~zero], want.view(np.uint16)[~zero]
    bad = np.nonzero(a != b)[0]
    assert bad.size == 0, f"{what}: {bad.size} weights differ, first at flat index {bad[0]}: {a[bad[0]]:#06x} vs {b[bad[0]]:#06x}"


@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("variant", [1, 3, 5, 6, 7, 9])
@pytest.mark.parametrize("expo", [False, True], ids=["linear", "mixed"])
def test_tile_kernels_return_the_dequantised_weights(H, bits, sparse, variant, expo):
    """`linear`: no exponent group anywhere, so the pipelined kernels run their linear-only loop;
    `mixed`: every tile holds groups of both modes and takes the loop (or, for the 128-column and
    16:32 tiles, the plain loop) that decodes either."""
    if variant == 5 and sparse:
        pytest.skip("256 x 128 tiles serve the dense formats only")
    K, S, g = 512, 512, 128
    p = _problem(bits, sparse, K, S, g, seed=70 + bits, expo=expo)
    want = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], g, p["sparse_mask"])
    d = H.dev_problem(p)
    H.capi.tune(3, variant)
    try:
        for split in (1, 2):                     # K never split / split in two where the variant can
            H.capi.tune(6, split)
            got = H.run_capi(p, d, "mtx", outs_init=np.full((1, K, S), 3.0, np.float16))
            _assert_same_bits(got[0], want, f"variant {variant} split {split}")
    finally:
        H.capi.tune(6, 0)
        H.capi.tune(3, 0)


@pytest.mark.parametrize("bits,sparse", FORMATS)
def test_default_dispatch_and_single_group(H, bits, sparse):
    # whatever kernel the launcher picks, more groups (g = 64), and the single-group mode
    for K, S, g in [(1024, 256, 64), (256, 768, -1)]:
        p = _problem(bits, sparse, K, S, 64 if g < 0 else g, seed=80 + bits)
        if g < 0:
            p = dict(p, group_size=-1, scales=p["scales"][:1].copy(), zeros=p["zeros"][:1].copy())
        want = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], p["group_size"], p["sparse_mask"])
        d = H.dev_problem(p)
        _assert_same_bits(H.run_capi(p, d, "mtx")[0], want, f"K={K} S={S} g={g}")


@pytest.mark.parametrize("bits,sparse", FORMATS)
@pytest.mark.parametrize("rows", [17, 64, 256])
def test_wide_rows_kernel_returns_the_dequantised_weights(H, bits, sparse, rows):
    K, S, g = 512, 512, 128
    p = _problem(bits, sparse, K, S, g, seed=90 + bits)
    want = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], g, p["sparse_mask"])
    H.capi.tune(8, 2)                            # the kernel with shared staging from 2 rows on, whatever the shape
    try:
        for r0 in (0, K - rows):
            q = dict(p, M=rows, states=np.ascontiguousarray(p["states"][:, r0:r0 + rows]))
            d = H.dev_problem(q)
            for split in (1, 0):                 # unsplit / the launcher's own choice
                H.capi.tune(6, split)
                got = H.run_capi(q, d, "mtx")
                _assert_same_bits(got[0], want[r0:r0 + rows], f"rows {r0}..{r0 + rows} split {split}")
    finally:
        H.capi.tune(6, 0)
        H.capi.tune(8, 0)


def test_helper_dequantise_matches_at_the_same_inputs(H):
    # the exported helper (the generic decode) and the matmul's fast decoders agree with each other too
    p = _problem(4, False, 512, 512, 128, seed=99)
    d = H.dev_problem(p)
    w = torch.empty((512, 512), dtype=torch.float16, device="cuda")
    H.capi.dequantize(4, w, d["matrix"], d["scales"], d["zeros"], 128, None)
    torch.cuda.synchronize()
    _assert_same_bits(H.run_capi(p, d, "mtx")[0], w.cpu().numpy(), "helper vs product")
