"""Pins the CPU oracle (oracle/w4a16_oracle.py, oracle/w4a16_oracle.c).

The reference holds no golden vectors for this path, so every oracle function is
pinned by hand-derived known answers (tests/golden/kat_handmade.json), by closed
forms, by exact (float64 / integer) arithmetic, by brute force against an
independent derivation, and by requiring the numpy and the C restatements to agree
bit for bit.
"""
import ctypes
import json
import os

from fractions import Fraction

import numpy as np
import pytest

import w4a16_oracle as orc

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat_handmade.json")))


# ---------------------------------------------------------------- unpack
def test_unpack_magic_exhaustive_closed_form():
    # every nibble value at every nibble position, others randomised
    rng = np.random.default_rng(0)
    for pos in range(8):
        for val in range(16):
            base = rng.integers(0, 2 ** 32, size=64, dtype=np.uint64).astype(np.uint32)
            w = (base & ~np.uint32(0xF << (4 * pos))) | np.uint32(val << (4 * pos))
            out = orc.unpack_u32_magic(w)
            for i, p in enumerate(orc.MAGIC_ORDER):
                expect = 64.0 + ((w >> np.uint32(4 * p)) & 0xF).astype(np.float32)
                assert np.array_equal(out[:, i].astype(np.float32), expect)


def test_unpack_magic_kat():
    k = KAT["unpack_magic"]
    out = orc.unpack_u32_magic(np.array([k["word"]], dtype=np.uint32))[0]
    assert out.astype(np.float32).tolist() == [float(v) for v in k["fp16_values"]]


def test_unpack_c_matches_numpy(oracle_c):
    rng = np.random.default_rng(1)
    words = rng.integers(0, 2 ** 32, size=2000, dtype=np.uint64).astype(np.uint32)
    ref = orc.unpack_u32_magic(words).view(np.uint16)
    buf = (ctypes.c_uint16 * 8)()
    for i, w in enumerate(words):
        oracle_c.sq_oracle_unpack8(ctypes.c_uint32(int(w)), buf)
        assert list(buf) == ref[i].tolist()


def test_c_half_conversions_all_patterns(oracle_c):
    # h2f on all 65536 patterns, and f2h(h2f(h)) == h for every non-NaN pattern
    for h in range(0, 65536, 1):
        f = oracle_c.sq_oracle_h2f(h)
        ref = np.array([h], dtype=np.uint16).view(np.float16)[0]
        if np.isnan(ref):
            assert np.isnan(f)
            continue
        assert f == np.float32(ref)
        assert oracle_c.sq_oracle_f2h(ctypes.c_float(f)) == h


def test_c_f2h_rounding_vs_numpy(oracle_c):
    rng = np.random.default_rng(2)
    vals = np.concatenate([
        rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000), rng.normal(0, 3e4, 2000),
        np.array([65504.0, 65519.9, 65520.0, 1e-8, 2.98e-8, 2.9802322e-08, 6.1e-5, -0.0, 0.0]),
    ]).astype(np.float32)
    for v in vals:
        got = oracle_c.sq_oracle_f2h(ctypes.c_float(float(v)))
        want = int(np.array([v], dtype=np.float32).astype(np.float16).view(np.uint16)[0])
        assert got == want, (v, got, want)


# ---------------------------------------------------------------- layout L1
def test_pack_l1_kat():
    k = KAT["l1_pack"]
    w = orc.pack_l1(np.array([k["q_row"]], dtype=np.uint8))
    assert w[0].tolist() == k["bytes"]


def test_pack_l1_roundtrip_and_natural_order():
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, size=(24, 256), dtype=np.uint8)
    w = orc.pack_l1(q)
    assert w.shape == (24, 128) and w.dtype == np.uint8
    assert np.array_equal(orc.unpack_l1(w), q)
    # the magic unpack of the packed words yields natural k order directly
    h = orc.unpack_u32_magic(np.ascontiguousarray(w).view(np.uint32)).reshape(24, 256)
    assert np.array_equal(h.astype(np.int32) - 64, q.astype(np.int32))


def test_zeros_scales_l1_kat_and_roundtrip():
    k = KAT["zeros_scales_l1"]
    zs = orc.zeros_scales_l1(np.array(k["zeros"]), np.array(k["scales"]))
    assert zs.dtype == np.float16 and zs.astype(np.float32).tolist() == [k["row"]]
    rng = np.random.default_rng(4)
    z = rng.integers(0, 16, size=(5, 7))
    s = rng.random((5, 7)).astype(np.float16)
    z64, s2 = orc.split_zeros_scales_l1(orc.zeros_scales_l1(z, s))
    assert np.array_equal(z64.astype(np.int32) - 64, z) and np.array_equal(s2, s)


def test_dequant_exact_arithmetic_all_q_z():
    # every (q, z) pair against many scales, expected value from exact float64
    # arithmetic rounded once to fp16
    rng = np.random.default_rng(5)
    scales = np.concatenate([
        (np.abs(rng.normal(0, 0.02, 60)) + 1e-3), np.array([1.0, 0.5, 0.1, 1e-3, 6.2e-5, 3e-6, 123.4])
    ]).astype(np.float16)
    qs = np.arange(16, dtype=np.uint8)
    for s in scales:
        for z in range(16):
            q = np.tile(qs, 2)[None, :]  # [1, 32]
            w = orc.pack_l1(q)
            zs = orc.zeros_scales_l1(np.array([[z]]), np.array([[s]]))
            got = orc.dequant_l1(w, zs, 32)[0]
            want = ((q[0].astype(np.float64) - z) * np.float64(s)).astype(np.float16)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (s, z)


def test_dequant_group_indexing():
    # distinct (z, s) per group: element k must use group k // g
    n, k, g = 3, 256, 64
    q = np.full((n, k), 9, dtype=np.uint8)
    z = np.arange(n * (k // g)).reshape(n, k // g) % 16
    s = (np.arange(n * (k // g)).reshape(n, k // g) + 1).astype(np.float16) / 8
    got = orc.dequant_l1(orc.pack_l1(q), orc.zeros_scales_l1(z, s), g).astype(np.float32)
    for r in range(n):
        for j in range(k // g):
            assert np.all(got[r, j * g:(j + 1) * g] == (9 - z[r, j]) * np.float32(s[r, j]))


def test_dequant_c_matches_numpy_bitwise(oracle_c):
    for g in (32, 64, 128):
        d = orc.synth_linear(48, 512, g, seed=g)
        ref = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
        out = np.empty((48, 512), dtype=np.uint16)
        oracle_c.sq_oracle_dequant_l1(d["w_l1"].ctypes.data_as(ctypes.c_void_p),
                                      d["zs_l1"].ctypes.data_as(ctypes.c_void_p),
                                      out.ctypes.data_as(ctypes.c_void_p), 48, 512, g)
        assert np.array_equal(out, ref.view(np.uint16))


# ---------------------------------------------------------------- layout L2
def test_ours_and_awq_kat():
    k = KAT["ours_pack"]
    assert orc.pack_ours(np.array([k["q_row"]], dtype=np.uint8))[0].tolist() == k["bytes"]
    a = KAT["awq_word"]
    q = np.zeros((8, 2), dtype=np.uint8)
    q[:, 0] = a["column_values_v0_to_v7"]
    q[:, 1] = a["column_values_v0_to_v7"]
    word = orc.ours_to_awq(orc.pack_ours(q), 2, 8)
    assert word.shape == (2, 1) and int(word[0, 0]) == a["word"] and int(word[1, 0]) == a["word"]


def test_lmdeploy_offset_kat():
    k = KAT["lmdeploy_offset"]
    for c in k["cases"]:
        assert orc.lmdeploy_nibble_offset(c["n"], c["k"], k["out_features"]) == c["offset"], c


@pytest.mark.parametrize("n,k", [(32, 32), (96, 64), (64, 160)])
def test_lmdeploy_bruteforce_permutation_matches_closed_form(n, k):
    rng = np.random.default_rng(n * 1000 + k)
    q = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
    w = orc.pack_l2(q)
    assert w.shape == (k, n // 8) and w.dtype == np.int32
    # closed form is a bijection onto [0, n*k)
    nn, kk = np.meshgrid(np.arange(n), np.arange(k), indexing="ij")
    off = orc.lmdeploy_nibble_offset(nn, kk, n).reshape(-1)
    assert np.array_equal(np.sort(off), np.arange(n * k))
    # and reading through it recovers q from the brute-force permuted storage
    assert np.array_equal(orc.unpack_l2(w, k, n), q)


def test_transpose_merge_zeros_scales_formula():
    n, k, g = 16, 512, 128
    rng = np.random.default_rng(7)
    z = rng.integers(0, 16, size=(n, k // g)).astype(np.float16)
    s = rng.random((n, k // g)).astype(np.float16)
    zs = orc.transpose_merge_zeros_scales(z, s, k, n, g)
    assert zs.shape == (k // g, 2 * n)
    flat = zs.reshape(-1, 2)
    for r in range(n):
        for j in range(k // g):
            assert flat[j * n + r, 0] == z[r, j] + np.float16(64) and flat[j * n + r, 1] == s[r, j]


def test_dequant_l2_equals_l1():
    n, k, g = 64, 256, 128
    d = orc.synth_linear(n, k, g, seed=11)
    zs2 = orc.transpose_merge_zeros_scales(d["z"].astype(np.float16), d["s"], k, n, g)
    a = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
    b = orc.dequant_l2(orc.pack_l2(d["q"]), zs2, g, k, n)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


# ---------------------------------------------------------------- GEMM
def test_gemm_ref_float64_and_onehot():
    n, k, g, m = 40, 256, 64, 5
    d = orc.synth_linear(n, k, g, seed=21)
    w_hat = orc.dequant_l1(d["w_l1"], d["zs_l1"], g)
    x = orc.synth_x(m, k, seed=22)
    y, y16 = orc.gemm_l1(x, d["w_l1"], d["zs_l1"], g)
    y64 = x.astype(np.float64) @ w_hat.astype(np.float64).T
    assert np.max(np.abs(y - y64)) <= 1e-4 * np.max(np.abs(y64))
    # a one-hot activation row picks a column of W_hat exactly
    e = np.zeros((1, k), dtype=np.float16)
    e[0, 77] = 1
    assert np.array_equal(orc.gemm_ref(e, w_hat)[0].astype(np.float16), w_hat[:, 77])
    # q == z gives an exactly zero output
    q = np.repeat(d["z"], g, axis=1).astype(np.uint8)
    y0, _ = orc.gemm_l1(x, orc.pack_l1(q), d["zs_l1"], g)
    assert np.all(y0 == 0)


def test_gemm_c_matches_numpy(oracle_c):
    n, k, g, m = 32, 512, 128, 3
    d = orc.synth_linear(n, k, g, seed=31)
    x = orc.synth_x(m, k, seed=32)
    y, _ = orc.gemm_l1(x, d["w_l1"], d["zs_l1"], g)
    out = np.empty((m, n), dtype=np.float32)
    oracle_c.sq_oracle_gemm_l1(x.ctypes.data_as(ctypes.c_void_p), d["w_l1"].ctypes.data_as(ctypes.c_void_p),
                               d["zs_l1"].ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
                               m, n, k, g)
    assert np.max(np.abs(out - y)) <= 2e-5 * np.max(np.abs(y))


# ---------------------------------------------------------------- either side
def test_rtn_kat():
    k = KAT["rtn"]
    q, s, z = orc.rtn_quantize(np.array(k["w"], dtype=np.float32), k["n_bit"], k["group"])
    assert q[0].tolist() == k["q"]
    assert abs(float(s[0, 0]) - k["scale"]) < 1e-6 and float(z[0, 0]) == k["zero"]


def _rn16(fr):
    """Exact rational -> nearest fp16 (ties to even), as a Fraction; written out bit by bit so that it does
    not lean on numpy's conversions."""
    from fractions import Fraction
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = 0
    while a >= 2:
        a /= 2
        e += 1
    while a < 1:
        a *= 2
        e -= 1
    e = max(e, -14)                      # subnormals share the exponent of the smallest normal
    ulp = Fraction(2) ** (e - 10)
    n = abs(fr) / ulp
    lo = n.numerator // n.denominator
    rem = n - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    if lo * ulp >= 65520:
        return Fraction(sign * 10 ** 9)   # overflow to infinity: any value that every later clamp saturates
    return sign * lo * ulp


def _round_half_even(fr):
    lo = fr.numerator // fr.denominator
    rem = fr - lo
    return lo + 1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1) else lo


def test_rtn_in_fp16_matches_exact_rational_arithmetic():
    """The quantiser in fp16 (what the reference computes on the fp16 weights it packs): every operation
    of the formula done in exact rational arithmetic and rounded to fp16 by hand."""
    rng = np.random.default_rng(43)
    w = rng.normal(0, 0.05, size=(6, 64)).astype(np.float16)
    w[1, :32] = np.float16(0.25)         # a constant group: the 1e-5 clamp
    differs = False
    for g in (32, 64):
        q, s, z = orc.rtn_quantize(w, 4, g, dtype=np.float16)
        q32, _, _ = orc.rtn_quantize(w.astype(np.float32), 4, g)
        differs |= not np.array_equal(q, q32)
        for r in range(w.shape[0]):
            for gi in range(64 // g):
                vals = [Fraction(float(v)) for v in w[r, gi * g:(gi + 1) * g]]
                d = max(_rn16(max(vals) - min(vals)), _rn16(Fraction(1e-5)))
                sc = _rn16(d / 15)
                assert Fraction(float(s[r, gi])) == sc
                zero = min(max(-_round_half_even(_rn16(min(vals) / sc)), 0), 15)
                assert int(z[r, gi]) == zero
                for j, v in enumerate(vals):
                    t = _rn16(v / sc)
                    want = min(max(_round_half_even(t) + zero, 0), 15)
                    assert int(q[r, gi * g + j]) == want, (r, gi, j)
    assert differs, "the fp16 and fp32 quantisers never disagreed: the test does not separate them"


def test_rtn_properties():
    rng = np.random.default_rng(41)
    w = rng.normal(0, 0.05, size=(16, 256)).astype(np.float32)
    q, s, z = orc.rtn_quantize(w, 4, 64)
    assert q.min() >= 0 and q.max() <= 15
    deq = (q.astype(np.float32) - np.repeat(z, 64, axis=1)) * np.repeat(s, 64, axis=1)
    assert np.max(np.abs(deq - w)) <= 0.5 * np.max(s) * 1.0001 + 1e-7
    # group extremes map to the ends of the code range
    assert np.all(q.reshape(16, 4, 64).max(axis=2) == 15)


def test_two_bit_kat_and_exhaustive():
    k = KAT["two_bit"]
    b = orc.pack_2bit_l1(np.array([k["values"]], dtype=np.uint8))
    assert b.tolist() == [[k["byte_2bit"]]]
    assert orc.convert_2bit_to_4bit_l1(b).tolist() == [k["bytes_4bit"]]
    # all 256 bytes: the four 2-bit fields land in four nibbles, order preserved
    allb = np.arange(256, dtype=np.uint8)[None, :]
    out = orc.convert_2bit_to_4bit_l1(allb)[0].reshape(256, 2)
    for v in range(256):
        a, bb, c, d = (v >> 4) & 3, (v >> 6) & 3, v & 3, (v >> 2) & 3
        assert out[v, 0] == (a | (bb << 4)) and out[v, 1] == (c | (d << 4))


def test_silu_dot_closed_forms():
    from scipy.special import expit
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, size=(3, 16))
    wg = rng.normal(0, 1, size=(5, 16))
    wu = rng.normal(0, 1, size=(5, 16))
    a, b = x @ wg.T, x @ wu.T
    got = orc.silu_dot_ref(x, wg, wu)
    assert np.allclose(got, a * expit(a) * b, rtol=1e-12, atol=1e-12)  # library logistic function
    # silu(a) - silu(-a) = a, so flipping the gate weight changes the result by exactly a * b
    assert np.allclose(got - orc.silu_dot_ref(x, -wg, wu), a * b, rtol=1e-12, atol=1e-12)
    # a zero gate gives zero; a saturated gate passes a * b (positive side) or nothing (negative side)
    assert np.all(orc.silu_dot_ref(x, np.zeros_like(wg), wu) == 0)
    g = orc.silu_dot_ref(np.eye(4), np.diag([40.0, -40.0, 0.0, 1.0]), 3.0 * np.eye(4))
    assert np.allclose(np.diag(g), [120.0, 0.0, 0.0, 3.0 / (1.0 + np.exp(-1.0))], atol=1e-12)
    # the two projections are not interchangeable
    assert not np.allclose(got, orc.silu_dot_ref(x, wu, wg))


def _int32_sum(terms):
    """Sum as torch's int32 `+=` gives it: modulo 2**32."""
    return sum(terms) & 0xFFFFFFFF


def _pack_pair_termwise(a, b):
    """The sixteen terms of the packer's loop, each parenthesised the way Python's grammar
    groups it (multiplication, then +/-, then shifts left to right, then &)."""
    terms = []
    for i in range(1, 9):
        terms.append(a & ((0x30000000 >> (4 * (i - 1))) << (2 * i)))
        terms.append(b & ((0x30000000 >> (4 * (i - 1))) >> (16 - 2 * i)))
    return _int32_sum(terms)


def _expand_termwise(w):
    first, second = [], []
    for i in range(1, 9):
        first.append(w & ((0xC0000000 >> (2 * (i - 1))) >> (2 * i)))
        second.append(w & ((0x0000C000 >> (2 * (i - 1))) << (16 - 2 * i)))
    return _int32_sum(first), _int32_sum(second)


def test_two_bit_int32_layout_words():
    """The int32-layout 2-bit pair computes what the reference's expressions compute under
    Python's precedence: checked term by term, on one-hot words and on a hand vector."""
    # Python really groups the unparenthesised source text this way.
    a, b, i = 0x89ABCDEF, 0x13579BDF, 3
    assert (a & (0x30000000 >> 4 * (i - 1)) << 2 * i) == (a & ((0x30000000 >> (4 * (i - 1))) << (2 * i)))
    assert (b & (0x30000000 >> 4 * (i - 1)) >> 16 - 2 * i) == (b & ((0x30000000 >> (4 * (i - 1))) >> (16 - 2 * i)))
    assert (a & (0xC0000000 >> 2 * (i - 1)) >> 2 * i) == (a & ((0xC0000000 >> (2 * (i - 1))) >> (2 * i)))
    assert (b & (0x0000C000 >> 2 * (i - 1)) << 16 - 2 * i) == (b & ((0x0000C000 >> (2 * (i - 1))) << (16 - 2 * i)))

    k = KAT["two_bit_int32"]
    w4 = np.array([k["words_4bit"]], dtype=np.uint32).view(np.int32)
    packed = orc.convert_4bit_to_2bit_l2(w4)
    assert packed.view(np.uint32).tolist() == [k["words_2bit"]]
    assert orc.convert_2bit_to_4bit_l2(packed).view(np.uint32).tolist() == [k["words_expanded"]]

    rng = np.random.default_rng(23)
    w = rng.integers(0, 2**32, size=(6, 8), dtype=np.uint64).astype(np.uint32)
    got = orc.convert_4bit_to_2bit_l2(w.view(np.int32)).view(np.uint32)
    assert got.shape == (6, 4)
    flat = w.reshape(-1, 2)
    want = [_pack_pair_termwise(int(p[0]), int(p[1])) for p in flat]
    assert got.reshape(-1).tolist() == want
    back = orc.convert_2bit_to_4bit_l2(got.view(np.int32)).view(np.uint32)
    assert back.shape == (6, 8)
    want_back = [x for v in got.reshape(-1) for x in _expand_termwise(int(v))]
    assert back.reshape(-1).tolist() == want_back

    # One-hot inputs: a bit of the first word survives iff it is in the upper half, a bit of the
    # second iff it is in the lower half, and it stays where it was.
    for bit in range(32):
        one = np.uint32(1 << bit)
        pa = orc.convert_4bit_to_2bit_l2(np.array([[one, 0]], dtype=np.uint32).view(np.int32)).view(np.uint32)[0, 0]
        pb = orc.convert_4bit_to_2bit_l2(np.array([[0, one]], dtype=np.uint32).view(np.int32)).view(np.uint32)[0, 0]
        assert pa == (one if bit >= 16 else 0) and pb == (one if bit < 16 else 0)
        e = orc.convert_2bit_to_4bit_l2(np.array([[one]], dtype=np.uint32).view(np.int32)).view(np.uint32)[0]
        keep = one if (bit % 4) < 2 else 0
        assert e.tolist() == [keep, keep]
    # Words holding 2-bit codes (every nibble <= 3): the upper four codes of the first word and the
    # lower four of the second come back; the other eight are replaced by their neighbours'.
    codes = rng.integers(0, 4, size=(5, 4, 8), dtype=np.uint32)
    words = (codes << (4 * np.arange(8, dtype=np.uint32))).sum(axis=2).astype(np.uint32)
    rt = orc.convert_2bit_to_4bit_l2(orc.convert_4bit_to_2bit_l2(words.view(np.int32))).view(np.uint32)
    rt_codes = (rt[..., None] >> (4 * np.arange(8, dtype=np.uint32))) & 15
    pairs = codes.reshape(5, 2, 2, 8)
    rtp = rt_codes.reshape(5, 2, 2, 8)
    assert np.array_equal(rtp[:, :, 0, 4:], pairs[:, :, 0, 4:]) and np.array_equal(rtp[:, :, 1, :4], pairs[:, :, 1, :4])
    assert np.array_equal(rtp[:, :, 0, :4], pairs[:, :, 1, :4]) and np.array_equal(rtp[:, :, 1, 4:], pairs[:, :, 0, 4:])


# ---- LayerNorm restatement ----

def test_layernorm_closed_forms():
    rng = np.random.default_rng(0)
    gamma = rng.normal(size=16)
    beta = rng.normal(size=16)
    # a constant row has zero deviation: the output is beta
    assert np.allclose(orc.layernorm_ref(np.full((2, 16), 3.25), gamma, beta), np.broadcast_to(beta, (2, 16)), atol=1e-12)
    # +-1 alternating: mean 0, variance 1
    x = np.tile([1.0, -1.0], 8)[None]
    assert np.allclose(orc.layernorm_ref(x, gamma, beta, eps=1e-5), x / np.sqrt(1 + 1e-5) * gamma + beta, atol=1e-12)
    # statistics by hand: [0, 0, 0, 4] has mean 1 and biased variance 3
    y = orc.layernorm_ref(np.array([[0.0, 0.0, 0.0, 4.0]]), eps=0.0)
    assert np.allclose(y, np.array([[-1.0, -1.0, -1.0, 3.0]]) / np.sqrt(3.0), atol=1e-12)
    # shift invariance, and unit variance / zero mean of the normalised row
    x = rng.normal(size=(3, 64))
    assert np.allclose(orc.layernorm_ref(x + 7.5, eps=1e-5), orc.layernorm_ref(x, eps=1e-5), atol=1e-9)
    y = orc.layernorm_ref(x, eps=0.0)
    assert np.allclose(y.mean(axis=-1), 0, atol=1e-12) and np.allclose((y ** 2).mean(axis=-1), 1, atol=1e-12)
