"""GPU parity, integer side: pack / unpack / dequantise kernels against the CPU
oracle, bit for bit, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

CASES = [(4, False), (3, False), (2, False), (4, True)]


@pytest.fixture(scope="module")
def H():
    from tests import helpers
    return helpers


@pytest.mark.parametrize("bits,sparse", CASES)
@pytest.mark.parametrize("K,S,g", [(64, 64, 64), (256, 320, 128), (1024, 1024, 64), (384, 64, -1)])
def test_dequantize_bit_exact(H, bits, sparse, K, S, g):
    p = O.make_problem(K=K, S=S, bits=bits, group_size=g, sparse=sparse, seed=K + S + bits)
    # mix in exponent-mode (negative scale) columns and groups
    p["scales"][:, ::3] *= np.float16(-1)
    d = H.dev_problem(p)
    out = torch.empty((K, S), dtype=torch.float16, device=H.DEV)
    H.capi.dequantize(bits, out, d["matrix"], d["scales"], d["zeros"], g, d["mask"])
    want = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], g, p["sparse_mask"])
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_dequantize_exhaustive_codes_and_zeros(H):
    """every int4 code x every fp16 zero in [0, 15] x 64 scales, both modes"""
    zbits = np.arange(0, int(np.float16(15).view(np.uint16)) + 1, dtype=np.uint16)
    n = (len(zbits) + 63) // 64 * 64
    zeros = np.zeros(n, np.float16)
    zeros[:len(zbits)] = zbits.view(np.float16)
    rng = np.random.default_rng(2)
    for sign in (1.0, -1.0):
        for srow in range(4):
            scales = (sign * rng.uniform(0.001, 1.01, n)).astype(np.float16)
            codes = np.tile(np.arange(16, dtype=np.uint8)[:, None], (4, n))      # K = 64
            matrix = O.pack_dense(4, codes)
            out = torch.empty((64, n), dtype=torch.float16, device=H.DEV)
            H.capi.dequantize(4, out, H.t(matrix), H.t(scales[None]), H.t(zeros[None]), 64, None)
            want = O.dequantize_matrix(4, matrix, scales[None], zeros[None], 64)
            assert np.array_equal(out.cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("bits,sparse", CASES)
def test_unpack_bit_exact(H, bits, sparse):
    K, S = 512, 192
    p = O.make_problem(K=K, S=S, bits=bits, sparse=sparse, seed=11 + bits)
    d = H.dev_problem(p)
    codes = torch.empty((K, S), dtype=torch.uint8, device=H.DEV)
    keep = torch.empty((K, S), dtype=torch.uint8, device=H.DEV)
    H.capi.unpack(bits, codes, keep, d["matrix"], d["mask"])
    assert np.array_equal(codes.cpu().numpy(), p["codes"])
    want_keep = p["keep"] if sparse else np.ones((K, S), bool)
    assert np.array_equal(keep.cpu().numpy().astype(bool), want_keep)


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_dense_pack_bit_exact_and_round_trip(H, bits):
    K, S = 640, 448
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, (K, S), dtype=np.uint8)
    out = torch.empty((K * bits // 32, S), dtype=torch.int32, device=H.DEV)
    H.capi.dense_pack(bits, out, H.t(codes))
    assert np.array_equal(out.cpu().numpy(), O.pack_dense(bits, codes))
    back = torch.empty((K, S), dtype=torch.uint8, device=H.DEV)
    H.capi.unpack(bits, back, None, out, None)
    assert np.array_equal(back.cpu().numpy(), codes)


def test_sparse_pack_bit_exact_capi_and_extension(H):
    S, K = 192, 1024
    p = O.make_problem(K=K, S=S, bits=4, sparse=True, seed=5)
    rng = np.random.default_rng(6)
    codes_sk = rng.integers(0, 16, (S, K), dtype=np.uint8)      # dropped rows carry junk codes
    keep_sk = np.ascontiguousarray(p["keep"].T).astype(np.uint8) * 3   # any value > 0 keeps
    want_w, want_m = O.sparse_pack(codes_sk, keep_sk)
    for via in ("capi", "ext"):
        w = torch.full((K // 16, S), -1, dtype=torch.int32, device=H.DEV)
        m = torch.full((K // 32, S), -1, dtype=torch.int32, device=H.DEV)
        if via == "capi":
            bad = torch.zeros(1, dtype=torch.int32, device=H.DEV)
            H.capi.sparse_pack(w, m, H.t(codes_sk), H.t(keep_sk), bad)
            assert int(bad.item()) == 0
        else:
            H.pkg.load_extension().weight_matrix_packing(w, m, H.t(codes_sk), H.t(keep_sk))
        assert np.array_equal(w.cpu().numpy(), want_w)
        assert np.array_equal(m.cpu().numpy(), want_m)


def test_sparse_pack_flags_wrong_popcount(H):
    S, K = 64, 64
    keep = np.zeros((S, K), np.uint8)
    keep[:, :16] = 1
    keep[:, 32:48] = 1
    keep[5, 40] = 0                       # one block keeps 15
    codes = np.zeros((S, K), np.uint8)
    w = torch.empty((K // 16, S), dtype=torch.int32, device=H.DEV)
    m = torch.empty((K // 32, S), dtype=torch.int32, device=H.DEV)
    bad = torch.zeros(1, dtype=torch.int32, device=H.DEV)
    H.capi.sparse_pack(w, m, H.t(codes), H.t(keep), bad)
    assert int(bad.item()) == 1
    with pytest.raises(RuntimeError):
        H.pkg.load_extension().weight_matrix_packing(w, m, H.t(codes), H.t(keep))


def test_sparse_pack_any_popcount_any_flag_value_high_code_bits(H):
    """the packer is rank based (utils_kernel.cu:29-63): a row is kept when its mask byte is > 0 (any value), only the
    low nibble of a code byte counts, the code of rank p < 16 lands at bits 4p and later ones are dropped -- checked
    cell by cell against that closed form for blocks keeping 0 ... 32 rows; S and K / 32 not multiples of the tile"""
    rng = np.random.default_rng(23)
    S, K = 70, 32 * 9
    codes = rng.integers(0, 256, (S, K), dtype=np.uint8)                       # high nibbles are noise
    prob = rng.random((S, K // 32, 1))
    keep = (rng.random((S, K // 32, 32)) < prob).astype(np.uint8) * rng.integers(1, 256, (S, K // 32, 32), dtype=np.uint8)
    keep[0, 0, :] = 0
    keep[1, 0, :] = 7
    keep = keep.reshape(S, K)
    w = torch.zeros((K // 16, S), dtype=torch.int32, device=H.DEV)
    m = torch.zeros((K // 32, S), dtype=torch.int32, device=H.DEV)
    bad = torch.zeros(1, dtype=torch.int32, device=H.DEV)
    H.capi.sparse_pack(w, m, H.t(codes), H.t(keep), bad)
    torch.cuda.synchronize()
    got_w = w.cpu().numpy().view(np.uint32)
    got_m = m.cpu().numpy().view(np.uint32)
    wrong = 0
    for s in range(S):
        for b in range(K // 32):
            bits, v, rank = 0, 0, 0
            for t in range(32):
                if keep[s, 32 * b + t] > 0:
                    bits |= 1 << t
                    if rank < 16:
                        v |= int(codes[s, 32 * b + t] & 0xF) << (4 * rank)
                    rank += 1
            wrong += rank != 16
            assert got_m[b, s] == bits, (s, b)
            assert got_w[2 * b, s] == (v & 0xFFFFFFFF) and got_w[2 * b + 1, s] == (v >> 32), (s, b)
    assert int(bad.item()) == wrong
