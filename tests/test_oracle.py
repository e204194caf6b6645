"""Pins the CPU oracle (oracle/oracle.py, oracle/oracle_c.c) without a GPU.

The reference holds no golden vectors or fixtures (its only test artefact is
the GPU script kernel_test.py), so the oracle is pinned by: hand-computed words
for single codes, the bit positions both reference decoders read, round trips,
agreement of two independently written restatements (closed-form numpy vs the
shift-and-consume C loops), exhaustive IEEE checks of the fp16 dequantisation,
and the harness's degenerate known-answer inputs (kernel_test.py:187-192,
210-215,242-243: every output equals K, or K/2 with 16:32 sparsity).
"""
from fractions import Fraction

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_c as OC


def u32(a):
    return np.ascontiguousarray(a).view(np.uint32)


# ---------------------------------------------------------------- fp16 helper
def test_c_half_conversion_matches_numpy_everywhere():
    L = OC.lib()
    allh = np.arange(65536, dtype=np.uint16)
    vals = allh.view(np.float16).astype(np.float64)
    for h, v in zip(allh[::7].tolist(), vals[::7].tolist()):
        got = L.oc_h2d(h)
        assert (np.isnan(v) and np.isnan(got)) or got == v
    rng = np.random.default_rng(1)
    d = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-9, 6, 20000),
                        # exact ties between neighbouring halves
                        (vals[1024:2048] + vals[1025:2049]) / 2,
                        [65504.0, 65519.999, 65520.0, 1e-8, 2.0 ** -25, 2.0 ** -24 * 1.5, 0.0, -0.0]])
    want = d.astype(np.float16).view(np.uint16)
    got = np.array([L.oc_d2h(float(x)) for x in d], dtype=np.uint16)
    assert np.array_equal(got, want)


# ------------------------------------------------------------- F1 / F2 dense
@pytest.mark.parametrize("bits", [4, 2])
def test_pow2_single_code_words(bits):
    per = 32 // bits
    K, S = 2 * per, 3
    for k in range(K):
        for v in (1, (1 << bits) - 1):
            codes = np.zeros((K, S), np.uint8)
            codes[k, 1] = v
            w = u32(O.pack_dense_pow2(bits, codes))
            expect = np.zeros((2, S), np.uint32)
            expect[k // per, 1] = v << (bits * (k % per))      # LSB-first field
            assert np.array_equal(w, expect)


def test_int4_top_nibble_is_negative_int32():
    codes = np.zeros((8, 1), np.uint8)
    codes[7, 0] = 9
    assert O.pack_dense_pow2(4, codes)[0, 0] == np.int32(-(1 << 32) + (9 << 28))


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_dense_round_trip_and_c_decoder(bits):
    rng = np.random.default_rng(bits)
    K, S = 192, 37
    codes = rng.integers(0, 1 << bits, (K, S), dtype=np.uint8)
    m = O.pack_dense(bits, codes)
    assert m.dtype == np.int32 and m.shape == (K * bits // 32, S)
    assert np.array_equal(O.unpack_dense(bits, m), codes)
    c2, keep = OC.unpack(bits, m, None, K)
    assert np.array_equal(c2, codes) and keep.all()


# ------------------------------------------------------------------ F3 int3
def _stream_words(codes32):
    """Independent statement with Python big ints: code j at stream bits 3j.."""
    s = 0
    for j, c in enumerate(codes32):
        s |= (int(c) & 7) << (3 * j)
    return [(s >> (32 * i)) & 0xFFFFFFFF for i in range(3)]


def test_int3_one_hot_positions():
    for j in range(32):
        for v in (1, 2, 4, 7):
            col = np.zeros((32, 1), np.uint8)
            col[j, 0] = v
            got = u32(O.pack_dense_int3(col))[:, 0].tolist()
            assert got == _stream_words(col[:, 0])


def test_int3_straddling_codes_hit_the_bits_the_decoders_read():
    # code 10: low 2 bits = top of word0, high bit = bit0 of word1
    # (matmul.cuh:289-292, matvec_kernel.cu:92-97)
    col = np.zeros((32, 1), np.uint8)
    col[10, 0] = 0b100
    assert u32(O.pack_dense_int3(col))[:, 0].tolist() == [0, 1, 0]
    col[10, 0] = 0b011
    assert u32(O.pack_dense_int3(col))[:, 0].tolist() == [0xC0000000, 0, 0]
    # code 21: low bit = bit31 of word1, high 2 bits = bits 0-1 of word2
    # (matmul.cuh:299-302, matvec_kernel.cu:107-111)
    col[:] = 0
    col[21, 0] = 0b001
    assert u32(O.pack_dense_int3(col))[:, 0].tolist() == [0, 0x80000000, 0]
    col[21, 0] = 0b110
    assert u32(O.pack_dense_int3(col))[:, 0].tolist() == [0, 0, 3]
    # code 11 starts at bit1 of word1, code 22 at bit2 of word2
    col[:] = 0
    col[11, 0] = 7
    col[22, 0] = 7
    assert u32(O.pack_dense_int3(col))[:, 0].tolist() == [0, 7 << 1, 7 << 2]


def test_int3_random_against_bigint_stream():
    rng = np.random.default_rng(33)
    codes = rng.integers(0, 8, (64, 5), dtype=np.uint8)
    w = u32(O.pack_dense_int3(codes))
    for s in range(5):
        for b in range(2):
            assert w[3 * b:3 * b + 3, s].tolist() == _stream_words(codes[32 * b:32 * b + 32, s])


# ---------------------------------------------------------------- F4 sparse
def _rand_keep(rng, S, K):
    keep = np.zeros((S, K // 32, 32), np.uint8)
    for s in range(S):
        for b in range(K // 32):
            keep[s, b, rng.permutation(32)[:16]] = 1
    return keep.reshape(S, K)


def test_sparse_fixed_masks_reduce_to_dense_int4():
    rng = np.random.default_rng(4)
    S, K = 7, 96
    codes = rng.integers(0, 16, (S, K), dtype=np.uint8)
    for lower in (True, False):
        keep = np.zeros((S, K // 32, 32), np.uint8)
        if lower:
            keep[:, :, :16] = 1
        else:
            keep[:, :, 16:] = 1
        keep = keep.reshape(S, K)
        wt, msk = O.sparse_pack(codes, keep)
        assert np.all(u32(msk) == (0x0000FFFF if lower else 0xFFFF0000))
        kept_rows = codes.T.reshape(K // 32, 32, S)[:, :16 if lower else None, :]
        kept_rows = kept_rows[:, :16, :] if lower else codes.T.reshape(K // 32, 32, S)[:, 16:, :]
        dense = O.pack_dense_pow2(4, kept_rows.reshape(K // 2, S))
        assert np.array_equal(wt, dense)


def test_sparse_pack_invariants_and_two_statements_agree():
    rng = np.random.default_rng(5)
    S, K = 9, 128
    codes = rng.integers(0, 16, (S, K), dtype=np.uint8)
    keep = _rand_keep(rng, S, K)
    wt, msk = O.sparse_pack(codes, keep)
    wt_c, msk_c, bad = OC.sparse_pack(codes, keep)
    assert bad == 0
    assert np.array_equal(wt, wt_c) and np.array_equal(msk, msk_c)
    pop = np.array([[bin(int(x)).count("1") for x in row] for row in u32(msk)])
    assert np.all(pop == 16)
    for dec in (lambda: O.sparse_unpack(wt, msk), lambda: OC.unpack(4, wt, msk, K)):
        c, k = dec()
        assert np.array_equal(k, keep.T.astype(bool))
        assert np.array_equal(c, (codes * keep).T)
    # mask bit t of block b <=> row 32b+t kept (ballot lane order, utils_kernel.cu:38)
    one = np.zeros((1, 32), np.uint8)
    one[0, [3] + list(range(17, 32))] = 1
    _, m1 = O.sparse_pack(np.zeros((1, 32), np.uint8), one)
    assert int(u32(m1)[0, 0]) == ((1 << 3) | 0xFFFE0000)


def test_sparse_pack_rejects_wrong_popcount():
    keep = np.zeros((1, 32), np.uint8)
    keep[0, :15] = 1
    with pytest.raises(ValueError):
        O.sparse_pack(np.zeros((1, 32), np.uint8), keep)
    assert OC.sparse_pack(np.zeros((1, 32), np.uint8), keep)[2] == 1


# ----------------------------------------------------------------- dequantise
def _round_half(fr: Fraction) -> np.float16:
    """Correctly rounded binary16 of an exact rational, via exact comparison."""
    if fr == 0:
        return np.float16(0)
    f = np.float64(fr.numerator) / np.float64(fr.denominator)
    c = np.float16(f)
    cands = {c, np.nextafter(c, np.float16(np.inf)), np.nextafter(c, np.float16(-np.inf))}
    best = sorted(cands, key=lambda h: (abs(Fraction(float(h)) - fr), int(np.float16(h).view(np.uint16)) & 1))
    return np.float16(best[0])


def test_dequant_linear_is_two_correctly_rounded_ops_exhaustive():
    # every fp16 zero in [0, 15], every int4 code, a sweep of scales
    zbits = np.arange(0, np.float16(15).view(np.uint16) + 1, dtype=np.uint16)
    z = zbits.view(np.float16)
    rng = np.random.default_rng(7)
    s = np.concatenate([rng.uniform(0.001, 0.02, 24), rng.uniform(0.01, 1.01, 8)]).astype(np.float16)
    q = np.arange(16, dtype=np.uint8)
    got = O.dequant_linear(q[:, None, None], s[None, None, :], z[None, :, None])
    # independent evaluation: exact double arithmetic, one rounding per op
    d = (q[:, None, None].astype(np.float64) - z[None, :, None].astype(np.float64)).astype(np.float16)
    want = (d.astype(np.float64) * s[None, None, :].astype(np.float64)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # exact rational spot checks of both roundings, and the scalar C path
    for qi, zi, si in [(0, 101, 0), (15, 19000, 3), (7, 18999, 30), (9, 17001, 12), (3, 15000, 25)]:
        zz, ss = z[zi], s[si]
        step1 = _round_half(Fraction(int(qi)) - Fraction(float(zz)))
        step2 = _round_half(Fraction(float(step1)) * Fraction(float(ss)))
        assert got[qi, zi, si].view(np.uint16) == step2.view(np.uint16)
        assert OC.dequant_scalar(qi, 4, ss, zz).view(np.uint16) == step2.view(np.uint16)


# Exponent quantisation, pinned by literal tables typed from the reference's text
# (matmul.cuh:127-136: iv = (v & SGN ? -1 : 1) * (1 << (v & EXP_MSK)), SGN = 1 << (bits - 1),
# EXP_MSK = SGN - 1, result = __hfma(half(iv), scale, zero); matmul.cuh:414-428: a stored scale
# below zero selects this branch and is negated first).  Every entry is an fp16 bit pattern worked
# out by hand; nothing here evaluates the oracle's own expression.
#   stored scale -0.5 (0xB800), zero 3.0 (0x4200): w = 3 + 0.5 * iv
EXPO_TABLE = {
    # iv:   +1      +2      +4      +8      +16     +32     +64     +128    -1      -2      -4      -8      -16     -32     -64     -128
    4: [0x4300, 0x4400, 0x4500, 0x4700, 0x4980, 0x4CC0, 0x5060, 0x5430, 0x4100, 0x4000, 0x3C00, 0xBC00, 0xC500, 0xCA80, 0xCF40, 0xD3A0],
    # iv:   +1      +2      +4      +8      -1      -2      -4      -8
    3: [0x4300, 0x4400, 0x4500, 0x4700, 0x4100, 0x4000, 0x3C00, 0xBC00],
    # iv:   +1      +2      -1      -2
    2: [0x4300, 0x4400, 0x4100, 0x4000],
}
#   int3, stored scale -0.75 (0xBA00), zero -1.25 (0xBD00): w = -1.25 + 0.75 * iv
#   = -0.5, 0.25, 1.75, 4.75, -2, -2.75, -4.25, -7.25
EXPO_TABLE_INT3_B = [0xB800, 0x3400, 0x3F00, 0x44C0, 0xC000, 0xC180, 0xC440, 0xC740]


def _h(bits16):
    return np.array(bits16, dtype=np.uint16).view(np.float16)


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_dequant_exponent_literal_table(bits):
    scale, zero = _h(0xB800), _h(0x4200)                  # -0.5, 3.0
    for v, want in enumerate(EXPO_TABLE[bits]):
        got = O.dequant_dynamic(bits, v, scale, zero)
        assert int(np.asarray(got).view(np.uint16)) == want, (bits, v)
        assert int(OC.dequant_scalar(v, bits, scale, zero).view(np.uint16)) == want, (bits, v)
        # the stand-alone exponent routine takes the already negated scale
        assert int(np.asarray(O.dequant_exponent(bits, v, _h(0x3800), zero)).view(np.uint16)) == want
    # bits above the field are ignored (the decoders hand over unmasked shifted words, matmul.cuh:131-134)
    assert int(np.asarray(O.dequant_dynamic(bits, (1 << bits) | 1, scale, zero)).view(np.uint16)) == EXPO_TABLE[bits][1]


def test_dequant_exponent_literal_table_int3_second_scale():
    scale, zero = _h(0xBA00), _h(0xBD00)                  # -0.75, -1.25
    for v, want in enumerate(EXPO_TABLE_INT3_B):
        assert int(np.asarray(O.dequant_dynamic(3, v, scale, zero)).view(np.uint16)) == want, v
        assert int(OC.dequant_scalar(v, 3, scale, zero).view(np.uint16)) == want, v


def test_dequant_exponent_is_one_fused_rounding_and_the_switch():
    # zero is ADDED (not subtracted) and the multiply-add rounds once:
    #   code 3 (iv = +8), stored scale -0.0999755859375 (0xAE66), zero 1000 (0x63D0):
    #   1000 + 0.7998046875 = 1000.7998..., fp16 spacing there is 0.5 -> 1001.0 = 0x63D2
    assert int(np.asarray(O.dequant_dynamic(4, 3, _h(0xAE66), _h(0x63D0))).view(np.uint16)) == 0x63D2
    assert int(OC.dequant_scalar(3, 4, _h(0xAE66), _h(0x63D0)).view(np.uint16)) == 0x63D2
    # no intermediate overflow: code 7 (iv = +128), stored scale -600 (0xE0B0), zero -60000 (0xFB53):
    # 76800 - 60000 = 16800 = 0x741A, although 76800 alone is beyond fp16 (a separate multiply gives inf)
    assert int(np.asarray(O.dequant_dynamic(4, 7, _h(0xE0B0), _h(0xFB53))).view(np.uint16)) == 0x741A
    assert int(OC.dequant_scalar(7, 4, _h(0xE0B0), _h(0xFB53)).view(np.uint16)) == 0x741A
    # the switch is `scale >= 0` (matmul.cuh:420): -0.0 stays linear: (5 - 1) * -0.0 = -0.0 = 0x8000;
    # +2.0 is linear: (5 - 1) * 2 = 8 = 0x4800; a NaN scale fails the comparison and takes the
    # exponent branch, whose result is NaN
    assert int(np.asarray(O.dequant_dynamic(4, 5, _h(0x8000), _h(0x3C00))).view(np.uint16)) == 0x8000
    assert int(OC.dequant_scalar(5, 4, _h(0x8000), _h(0x3C00)).view(np.uint16)) == 0x8000
    assert int(np.asarray(O.dequant_dynamic(4, 5, _h(0x4000), _h(0x3C00))).view(np.uint16)) == 0x4800
    assert np.isnan(float(O.dequant_dynamic(4, 5, _h(0x7E00), _h(0x3C00))))
    assert np.isnan(float(OC.dequant_scalar(5, 4, _h(0x7E00), _h(0x3C00))))


@pytest.mark.parametrize("bits,sparse", [(4, False), (3, False), (2, False), (4, True)])
def test_dequantize_matrix_two_statements_agree(bits, sparse):
    p = O.make_problem(K=256, S=24, bits=bits, group_size=64, sparse=sparse, seed=bits + 10)
    p["scales"][1, ::5] *= np.float16(-1)          # exercise the exponent branch too
    a = O.dequantize_matrix(bits, p["matrix"], p["scales"], p["zeros"], 64, p["sparse_mask"])
    b = OC.dequantize(bits, p["matrix"], p["scales"], p["zeros"], 64, p["sparse_mask"], 256)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    if sparse:
        assert np.all(a[~p["keep"]].view(np.uint16) == 0)      # exactly +0.0
        assert np.all(p["keep"].reshape(8, 32, 24).sum(1) == 16)


def test_group_size_minus_one_and_1d_params():
    p = O.make_problem(K=128, S=8, bits=4, group_size=-1, seed=3)
    assert p["scales"].shape == (1, 8)
    a = O.dequantize_matrix(4, p["matrix"], p["scales"], p["zeros"], -1)
    b = O.dequantize_matrix(4, p["matrix"], p["scales"][0], p["zeros"][0], -1)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    want = O.dequant_linear(p["codes"], p["scales"][0][None, :], p["zeros"][0][None, :])
    assert np.array_equal(a.view(np.uint16), want.view(np.uint16))


# ------------------------------------------------------------------- products
@pytest.mark.parametrize("bits,sparse,K", [(4, False, 5120), (3, False, 1024), (2, False, 1024),
                                           (4, True, 16384)])
def test_degenerate_known_answer(bits, sparse, K):
    """All-ones codes, zero zero-points, unit scales, all-ones states: every
    output is K (dense) or K/2 (sparse keeps 16 of 32) -- exact in fp16."""
    S = 64
    codes = np.ones((K, S), np.uint8)
    scales = np.ones((K // 128, S), np.float16)
    zeros = np.zeros((K // 128, S), np.float16)
    x = np.ones((1, 1, K), np.float16)
    if sparse:
        keep = np.zeros((S, K // 32, 32), np.uint8)
        keep[:, :, 16:] = 1                       # kernel_test.py:211-214 keeps one half
        matrix, mask = O.sparse_pack(np.ascontiguousarray(codes.T), keep.reshape(S, K))
    else:
        matrix, mask = O.pack_dense(bits, codes), None
    w16 = O.dequantize_matrix(bits, matrix, scales, zeros, 128, mask)
    y = O.matmul_exact(x[0], w16)
    want = K // 2 if sparse else K
    assert np.all(y == want)
    got = OC.matvec(bits, matrix, mask, x, scales, zeros, 128, np.zeros(S, np.float16))
    assert np.all(got.astype(np.float64) == want)


def test_matvec_port_accumulates_onto_outs_and_matches_exact():
    p = O.make_problem(K=1024, S=64, bits=4, group_size=64, seed=0)
    w16 = O.dequantize_matrix(4, p["matrix"], p["scales"], p["zeros"], 64)
    y = O.matmul_exact(p["states"][0], w16)[0]
    prior = np.linspace(-2, 2, 64).astype(np.float16)
    got = OC.matvec(4, p["matrix"], None, p["states"], p["scales"], p["zeros"], 64, prior)
    want = O.matvec_expected(prior, y)
    assert O.max_rel_error(want, got) < 2e-3
    w32 = O.dequantize_matrix_fp32(4, p["matrix"], p["scales"], p["zeros"], 64)
    assert O.max_rel_error(O.matmul_fp32(p["states"][0], w32)[0] + prior.astype(np.float32), got) < 1e-2
    assert O.mean_rel_error(O.matmul_fp32(p["states"][0], w32)[0] + prior.astype(np.float32), got) < 0.1


def test_metrics():
    t = np.array([1.0, 2.0, 0.0, 4.0])
    c = np.array([1.1, 2.0, 0.0, 4.0])
    assert abs(O.mean_rel_error(t, c) - 0.1 / 3) < 1e-12          # 0/0 is dropped by nanmean
    rms = np.sqrt(21 / 4)
    assert abs(O.max_rel_error(t, c) - 0.1 / rms) < 1e-12
    assert abs(O.max_rel_error(t, c, floor_frac=0.0) - 0.1) < 1e-9
