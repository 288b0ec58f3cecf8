"""Pins the CPU oracle.  The reference ships no tests, golden vectors or
fixtures for this path, so every function is checked against what the
mathematics fixes: closed forms, library routines (scipy.linalg.hadamard /
block_diag), brute force on small sizes, hand-derived tables, published
known-answer vectors (Philox, Random123) and statistical properties.  None of
the checks re-types the oracle's own formula."""
import itertools
import os

import numpy as np
from dataclasses import replace
import pytest
import scipy.linalg

from oracle import hot_oracle as orc

F32 = np.float32


# ------------------------------------------------------------------ sizes

def test_pow2_factor_bruteforce():
    for size in range(1, 400):
        best = max(d for d in range(1, size + 1) if size % d == 0 and (d & (d - 1)) == 0)
        assert orc.pow2_factor(size) == best
        assert orc.pow2_factor_max16(size) == (16 if best > 16 and size > 16 else best)


def test_pow2_factor_table():
    # sizes of the graded configurations
    assert [orc.pow2_factor_max16(v) for v in (768, 2304, 3072, 4096, 11008)] == [16] * 5
    assert orc.pow2_factor(12608) == 64 and orc.pow2_factor(8192) == 8192
    assert orc.pow2_factor(197) == 1 and orc.pow2_factor(49) == 1 and orc.pow2_factor(25216) == 128
    assert orc.pow2_factor_max16(16) == 16 and orc.pow2_factor_max16(8) == 8 and orc.pow2_factor_max16(12) == 4


# --------------------------------------------------------------- matrices

@pytest.mark.parametrize("n", [1, 2, 4, 8, 16, 32, 64, 128])
def test_hadamard_is_sylvester(n):
    H = orc.hadamard(n)
    if n > 1:
        assert np.array_equal(H, scipy.linalg.hadamard(n))
    assert np.array_equal(H, H.T)
    assert np.array_equal(H @ H.T, n * np.eye(n, dtype=np.int64))


def test_hadamard_rejects_non_power_of_two():
    for bad in (0, 3, 12, -4):
        with pytest.raises(ValueError):
            orc.hadamard(bad)


@pytest.mark.parametrize("n", [1, 2, 4, 8, 16, 32, 64, 128, 256])
def test_sequency_bruteforce(n):
    H = scipy.linalg.hadamard(n) if n > 1 else np.array([[1]])
    changes = np.array([(H[i, :-1] != H[i, 1:]).sum() for i in range(n)])
    assert np.array_equal(orc.sequency_of_natural(n), changes)
    assert sorted(changes) == list(range(n))          # unique: the sort is unambiguous
    assert np.array_equal(orc.sequency_of_natural(n)[orc.natural_of_sequency(n)], np.arange(n))


def test_kept_sequencies_hand_derived():
    # derived by hand from the band rule: band i of width s keeps its first s-i
    # entries when i is even and its last s-i entries when i is odd
    assert list(orc.kept_sequencies(1)) == [0]
    assert list(orc.kept_sequencies(2)) == [0]
    assert list(orc.kept_sequencies(4)) == [0, 1, 3]
    assert list(orc.kept_sequencies(8)) == [0, 1, 3]
    assert list(orc.kept_sequencies(16)) == [0, 1, 2, 3, 5, 6, 7, 8, 9, 15]
    k64 = list(orc.kept_sequencies(64))
    assert k64 == (list(range(0, 8)) + list(range(9, 16)) + list(range(16, 22)) + list(range(27, 32))
                   + list(range(32, 36)) + list(range(45, 48)) + list(range(48, 50)) + [63])
    for n, r in ((32, 10), (64, 36), (128, 36), (256, 136), (2048, 528), (4096, 2080), (8192, 2080)):
        assert len(orc.kept_sequencies(n)) == r


@pytest.mark.parametrize("size", [16, 48, 64, 192, 12608 // 197 * 3])
def test_make_wht_bruteforce(size):
    """P = rows of the Sylvester matrix sorted by counted sign changes, then the
    hand-derived index set."""
    n = orc.pow2_factor(size)
    H = scipy.linalg.hadamard(n) if n > 1 else np.array([[1]])
    order = sorted(range(n), key=lambda i: int((H[i, :-1] != H[i, 1:]).sum()))
    want = H[order][orc.kept_sequencies(n)]
    P = orc.make_WHT(size)
    assert np.array_equal(P, want)
    r = P.shape[0]
    assert np.array_equal(P @ P.T, n * np.eye(r, dtype=np.int64))


def test_vit_and_llama_token_rules():
    n, rows = orc.hla_rows(12608)
    assert (n, len(rows)) == (64, 36)
    n, rows = orc.hla_rows(8192)
    assert (n, len(rows)) == (8192, 2080)
    n, rows = orc.hla_rows(197)
    assert (n, list(rows)) == (1, [0])
    n, rows = orc.paper_rows(16, 8)
    H = scipy.linalg.hadamard(16)
    assert sorted(int((H[i, :-1] != H[i, 1:]).sum()) for i in rows) == list(range(8))


# -------------------------------------------------------------- transforms

@pytest.mark.parametrize("n", [2, 16, 32, 64])
def test_fwht_blocks_last_vs_blockdiag(n):
    rng = np.random.default_rng(n)
    a = rng.integers(-100, 100, size=(7, 3 * n)).astype(F32)      # exact in fp32
    bd = scipy.linalg.block_diag(*[orc.hadamard(n)] * 3).astype(F32)
    assert np.array_equal(orc.fwht_blocks_last(a, n), a @ bd)


@pytest.mark.parametrize("n", [1, 4, 16, 64])
def test_fwht_blocks_first_vs_blockdiag(n):
    rng = np.random.default_rng(n)
    a = rng.integers(-100, 100, size=(3 * n, 5)).astype(F32)
    bd = scipy.linalg.block_diag(*[orc.hadamard(n)] * 3).astype(F32)
    assert np.array_equal(orc.fwht_blocks_first(a, n), bd @ a)
    _, rows = orc.hla_rows(n) if n > 1 else (1, np.array([0]))
    P = orc.hadamard(n)[rows].astype(F32)
    bdp = scipy.linalg.block_diag(*[P] * 3)
    assert np.array_equal(orc.fwht_blocks_first(a, n, rows), bdp @ a)


def test_fwht_is_the_canonical_butterfly():
    """Stage order h = 1, 2, 4, 8 with (x+y, x-y), evaluated by a scalar loop."""
    rng = np.random.default_rng(0)
    v = rng.standard_normal(16).astype(F32)
    w = v.copy()
    h = 1
    while h < 16:
        for j in range(16):
            if (j // h) % 2 == 0:
                x, y = w[j], w[j + h]
                w[j], w[j + h] = F32(x + y), F32(x - y)
        h *= 2
    assert np.array_equal(orc.fwht_blocks_last(v[None, :], 16)[0], w)


def test_transform_rejects_ragged():
    with pytest.raises(ValueError):
        orc.fwht_blocks_last(np.zeros((2, 40), F32), 16)
    with pytest.raises(ValueError):
        orc.fwht_blocks_first(np.zeros((40, 2), F32), 16)


# ------------------------------------------------------------------ Philox

def test_philox_known_answers():
    """Random123 kat_vectors, philox4x32-10."""
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
         (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in kat:
        got = orc.philox4x32(*[[c] for c in ctr], key[0], key[1])
        assert tuple(int(g[0]) for g in got) == want


def test_sr_uniform_range_and_moments():
    u = orc.sr_uniform(np.arange(1 << 16), seed=12345, stream=1)
    assert u.dtype == F32 and u.min() >= 0.0 and u.max() < 1.0
    assert abs(u.mean() - 0.5) < 0.005 and abs(u.var() - 1 / 12) < 0.003
    hist = np.histogram(u, bins=16, range=(0, 1))[0]
    assert np.all(np.abs(hist - 4096) < 5 * 64)
    # different seeds / streams / indices give different draws
    assert not np.array_equal(u, orc.sr_uniform(np.arange(1 << 16), seed=12346, stream=1))
    assert not np.array_equal(u, orc.sr_uniform(np.arange(1 << 16), seed=12345, stream=2))
    assert np.array_equal(u[4:8], orc.sr_uniform(np.arange(4, 8), seed=12345, stream=1))
    # elements 8 q .. 8 q + 7 share Philox call q: low half of word 0, high half of word 0, low half of word 1, ...
    w = orc.philox4x32(np.array([5], np.uint64), np.array([0], np.uint64), np.array([1], np.uint64),
                       np.array([0], np.uint64), 12345, 0, rounds=orc.SR_PHILOX_ROUNDS)
    halves = []
    for i in range(4):
        halves += [int(w[i][0]) & 0xFFFF, int(w[i][0]) >> 16]
    assert np.array_equal(u[40:48], (np.array(halves, dtype=np.float32) / np.float32(65536.0)))


def test_philox_rounds_are_one_round_function_iterated():
    """The generator of stochastic rounding runs 7 rounds of the function whose 10-round form the known
    answers pin: a scalar restatement of one round (two 32 x 32 -> 64 products, the key bumped by the
    Weyl constants) applied r times equals philox4x32(rounds=r) for r = 1, 7 and 10."""
    def rounds(c, k, n):
        c, k = list(c), list(k)
        for _ in range(n):
            p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
            c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
            k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
        return tuple(c)
    assert orc.SR_PHILOX_ROUNDS == 7
    for ctr, key in (((0, 0, 0, 0), (0, 0)), ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0)),
                     ((123456789, 7, 3, 0), (42, 99))):
        for n in (1, 7, 10):
            got = orc.philox4x32(*[[c] for c in ctr], key[0], key[1], rounds=n)
            assert tuple(int(g[0]) for g in got) == rounds(ctr, key, n)
    assert rounds((0, 0, 0, 0), (0, 0), 10) == (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)


def _fma32(a, b, c):
    """fl32(a * b + c) for positive results, by exact rational arithmetic and one round-half-even to 24 bits"""
    from fractions import Fraction
    v = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
    e = v.numerator.bit_length() - v.denominator.bit_length()
    if Fraction(2) ** e > v:
        e -= 1
    ulp = Fraction(2) ** (e - 23)
    return float(round(v / ulp) * ulp)


def test_sr_codes_fixed_point_form():
    """sr_round: p = fma(|t|, fl32(1/d) 2^16, 0.5) in fp32, q = (trunc(p) + r) >> 16.  (a) the float64
    evaluation of the fused multiply-add equals exact rational arithmetic rounded once; (b) over all 65536
    values of r the number of round-ups is round(frac(|t| / d) 2^16) up to the 1.5 ulp of the reciprocal
    product, so the expectation is t / d within 2^-15; (c) codes are floor or ceil of |t / d|, carry the
    sign of t, never pass qmax, and zero stays zero."""
    rng = np.random.default_rng(7)
    t = np.concatenate([rng.standard_normal(300).astype(F32) * F32(3e-3), F32([0.0, 1e-30, -1e-30, 7e-3, -7e-3, 2.5e-7])])
    d = F32(F32(np.abs(t).max()) / F32(7) + F32(1e-11))
    rcpk = F32(F32(1.0) / d) * F32(65536.0)
    p_ref = np.array([_fma32(abs(float(v)), float(rcpk), 0.5) for v in t])
    p64 = (np.abs(t).astype(np.float64) * np.float64(rcpk) + 0.5).astype(F32)
    assert np.array_equal(p64.astype(np.float64), p_ref)
    y = np.abs(t.astype(np.float64)) / float(d)
    lo = orc.sr_round(t, d, 7, np.zeros(t.shape, np.uint32))
    hi = orc.sr_round(t, d, 7, np.full(t.shape, 65535, np.uint32))
    assert np.all((np.abs(lo) == np.floor(y + 2.0 ** -17)) | (np.abs(lo) == np.floor(y)))
    assert np.all(np.abs(hi) <= 7) and np.all(np.abs(hi) - np.abs(lo) <= 1) and np.all(np.abs(hi) >= np.abs(lo))
    assert np.all(np.sign(lo[lo != 0]) == np.sign(t[lo != 0])) and lo[300] == 0 and hi[300] == 0
    # the number of r that round up, counted exactly: the low 16 bits of trunc(p)
    ups = np.trunc(p_ref).astype(np.int64) & 0xFFFF
    frac16 = (y - np.floor(y)) * 65536.0
    wrap = np.minimum(np.abs(ups - frac16), 65536 - np.abs(ups - frac16))       # a fraction next to 1 rounds up into the next integer
    assert np.all(wrap <= 0.5 + 8 * 1.5 * 2.0 ** -24 * 65536 + 1e-6)
    for i in (0, 17, 303):
        r_all = np.arange(65536, dtype=np.uint32)
        q = orc.sr_round(np.full(65536, t[i], F32), d, 7, r_all)
        assert int((np.abs(q) != np.abs(lo[i])).sum()) == int(ups[i]) or abs(int(lo[i])) == 7
        assert abs(np.abs(q).mean() - y[i]) <= 2.0 ** -15
    # the top of the range: |t| = absmax is qmax (1 - a few ulp): qmax for all but the smallest few r, never more
    top = t[np.abs(t).argmax()]
    q = orc.sr_round(np.full(65536, top, F32), d, 7, np.arange(65536, dtype=np.uint32))
    assert np.abs(q).max() == 7 and int((np.abs(q) != 7).sum()) <= 16


# --------------------------------------------------------------- quantisers

def test_quant_nearest_ties_to_even():
    # mx = 7, bits = 4 -> s = 1, fl32(1 + 1e-11) = 1 -> y = t exactly
    t = np.array([[0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 6.5, 7.0, 0.49999997, 0.50000006]], F32)
    q, s = orc.quant(t, 4, orc.SCALE_TENSOR)
    assert s[0] == 1.0
    assert q.tolist() == [[0, 2, 2, 4, 0, -2, -2, 6, 7, 0, 1]]
    t8 = np.array([[127.0, 0.5, 1.5, -126.5, 63.5]], F32)
    q, s = orc.quant(t8, 8, orc.SCALE_TENSOR)
    assert s[0] == 1.0 and q.tolist() == [[127, 0, 2, -126, 64]]


def test_quant_zero_tensor_and_max():
    q, s = orc.quant(np.zeros((3, 8), F32), 4, orc.SCALE_TENSOR)
    assert not q.any() and s[0] == 0
    q, s = orc.quant(np.zeros((3, 8), F32), 8, orc.SCALE_ROW)
    assert not q.any() and not s.any() and s.shape == (3,)
    rng = np.random.default_rng(1)
    for bits in (4, 8):
        qm = 2 ** (bits - 1) - 1
        t = rng.standard_normal((40, 64)).astype(F32) * F32(1e-3)
        q, s = orc.quant(t, bits, orc.SCALE_TENSOR)
        i = np.unravel_index(np.argmax(np.abs(t)), t.shape)
        assert abs(int(q[i])) == qm and np.abs(q).max() == qm
        assert s[0] == F32(np.abs(t).max()) / F32(qm)
        # textbook absmax quantiser: reconstruction within half a step
        assert np.all(np.abs(q.astype(np.float64) * float(s[0]) - t) <= 0.5 * float(s[0]) * (1 + 1e-5))
        qr, sr = orc.quant(t, bits, orc.SCALE_ROW)
        assert np.all(np.abs(qr).max(axis=1) == qm)
        for r in (0, 17, 39):                      # rows are independent
            q1, s1 = orc.quant(t[r:r + 1], bits, orc.SCALE_TENSOR)
            assert np.array_equal(q1[0], qr[r]) and s1[0] == sr[r]


def test_quant_stochastic_statistics():
    rng = np.random.default_rng(2)
    t = rng.standard_normal((16, 64)).astype(F32)
    s, _ = orc.quant_scale(t, 4, orc.SCALE_TENSOR)
    y = (t / (s + F32(1e-11))).astype(np.float64)
    nseed = 600
    acc = np.zeros_like(y)
    acc2 = np.zeros_like(y)
    for seed in range(nseed):
        q, s2 = orc.quant(t, 4, orc.SCALE_TENSOR, orc.ROUND_STOCH, seed=seed, stream=0)
        q = q.astype(np.float64)
        assert np.all((q == np.floor(y)) | (q == np.ceil(y)))
        assert np.abs(q).max() <= 7 and s2[0] == s
        acc += q
        acc2 += q * q
    mean = acc / nseed
    assert np.max(np.abs(mean - y)) < 0.11                       # 5 sigma of 0.5 / sqrt(600)
    assert abs((mean - y).mean()) < 5 * 0.5 / np.sqrt(nseed * y.size)
    p = y - np.floor(y)
    var = acc2 / nseed - mean ** 2
    assert abs(var.mean() - (p * (1 - p)).mean()) < 0.01          # Bernoulli variance


def test_quant_sawb_closed_form():
    rng = np.random.default_rng(3)
    t = rng.standard_normal((64, 64)).astype(F32) * F32(0.02)
    q, s = orc.quant(t, 4, orc.SCALE_SAWB)
    clip = 12.1 * np.sqrt((t.astype(np.float64) ** 2).mean()) - 12.2 * np.abs(t.astype(np.float64)).mean()
    assert abs(float(s[0]) - clip / 7) < 1e-7 * clip
    # Gaussian data: clip = (12.1 - 12.2 sqrt(2/pi)) sigma ~ 2.37 sigma
    assert 2.2 * 0.02 < clip < 2.55 * 0.02
    assert np.abs(q).max() == 7
    inside = np.abs(t) < clip * 0.99
    assert np.all(np.abs(q[inside] * float(s[0]) - t[inside]) <= 0.5 * float(s[0]) * (1 + 1e-4))


# ------------------------------------------------------------- wire format

def test_int4_pack_all_pairs():
    pairs = np.array(list(itertools.product(range(-7, 8), repeat=2)), dtype=np.int8)   # 225 pairs
    assert pairs.shape == (225, 2)
    packed = orc.pack_int4(pairs)
    assert packed.shape == (225, 1)
    for (lo, hi), byte in zip(pairs.tolist(), packed.view(np.uint8)[:, 0].tolist()):
        assert byte == (((hi & 0xF) << 4) | (lo & 0xF))
    assert np.array_equal(orc.unpack_int4(packed), pairs)
    assert orc.pack_int4(np.array([[-1, 3]], np.int8)).view(np.uint8)[0, 0] == 0x3F
    assert orc.pack_int4(np.array([[7, -7]], np.int8)).view(np.uint8)[0, 0] == 0x97
    with pytest.raises(ValueError):
        orc.pack_int4(np.zeros((1, 3), np.int8))


def test_int_gemm_exact():
    rng = np.random.default_rng(4)
    a = rng.integers(-127, 128, size=(33, 700), dtype=np.int8)
    b = rng.integers(-127, 128, size=(21, 700), dtype=np.int8)
    assert np.array_equal(orc.int_gemm_nt(a, b), a.astype(np.int64) @ b.astype(np.int64).T)
    full = np.full((4, 11008), 127, np.int8)
    assert np.all(orc.int_gemm_nt(full, -full) == -127 * 127 * 11008)


# ------------------------------------------------------- the composed path

def _case(L=128, O=64, I=48, seed=0, outliers=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((L, I)).astype(F32)
    w = (rng.uniform(-1, 1, (O, I)) / np.sqrt(I)).astype(F32)
    gy = (rng.standard_normal((L, O)) * 1e-3).astype(F32)
    if outliers:
        gy = np.where(rng.uniform(size=gy.shape) < 0.01, gy * 50, gy).astype(F32)
    return x, w, gy


def _rel(a, b):
    return np.linalg.norm(a.astype(np.float64) - b) / np.linalg.norm(b)


def test_transforms_alone_are_exact():
    """H_n H_n^T = n I: without quantisation the path reproduces g_y W and, with
    all rows kept, g_y^T x (integer-valued inputs make fp32 exact)."""
    rng = np.random.default_rng(5)
    gy = rng.integers(-8, 8, (64, 32)).astype(F32)
    w = rng.integers(-8, 8, (32, 24)).astype(F32)
    x = rng.integers(-8, 8, (64, 24)).astype(F32)
    G, Wh = orc.fwht_blocks_last(gy, 16), orc.fwht_blocks_first(w, 16)
    assert np.array_equal(G @ Wh / 16, gy @ w)
    Gp = orc.fwht_blocks_first(gy, 16, np.arange(16))
    Xp = orc.fwht_blocks_first(x, 16, np.arange(16))
    assert np.array_equal(Gp.T @ Xp / 16, gy.T @ x)


def test_backward_int8_full_rank_is_close_to_fp():
    x, w, gy = _case()
    cfg = orc.HotConfig(hla_n=16, hla_rows=tuple(range(16)), gx_bits=8, w_bits=8, gw_bits=8, act_bits=8)
    xq, sx = orc.abc_forward(x, cfg)
    tr = orc.linear_backward(gy, w, xq, sx, cfg)
    assert _rel(tr.g_x, gy.astype(np.float64) @ w) < 0.02
    assert _rel(tr.g_w, gy.astype(np.float64).T @ x) < 0.02
    assert np.array_equal(tr.acc_x, tr.qG.astype(np.int64) @ tr.qW.astype(np.int64))
    assert np.array_equal(tr.acc_w, tr.qGp.astype(np.int64) @ xq.astype(np.int64))
    assert tr.g_x.shape == (128, 48) and tr.g_w.shape == (64, 48)


def test_hadamard_spreads_outliers():
    """INT8 g_x error with 1 % x50 outliers is lower (here about 3x) with the
    Hadamard transform than when quantising g_y and W directly."""
    x, w, gy = _case(L=256, O=128, I=64, seed=7, outliers=True)
    cfg = orc.HotConfig.python_rule(256, gx_bits=8, w_bits=8)
    xq, sx = orc.abc_forward(x, cfg)
    tr = orc.linear_backward(gy, w, xq, sx, cfg)
    exact = gy.astype(np.float64) @ w
    qg, sg = orc.quant(gy, 8, orc.SCALE_TENSOR)
    qw, sw = orc.quant(w.T.copy(), 8, orc.SCALE_TENSOR)
    plain = orc.int_gemm_nt(qg, qw).astype(np.float64) * float(sg[0]) * float(sw[0])
    assert _rel(tr.g_x, exact) < 0.6 * _rel(plain, exact)


def test_backward_low_rank_is_a_projection():
    """g_W of the low-rank path equals (P g_y)^T (P x) / n up to quantisation."""
    x, w, gy = _case(L=128, seed=9)
    cfg = orc.HotConfig.python_rule(128)
    n, rows = orc.hla_rows(128)
    assert cfg.hla_n == n == 128 and len(rows) == 36
    cfg8 = orc.HotConfig(hla_n=n, hla_rows=tuple(rows), gw_bits=8, act_bits=8)
    xq, sx = orc.abc_forward(x, cfg8)
    tr = orc.linear_backward(gy, w, xq, sx, cfg8)
    P = orc.make_WHT(128).astype(np.float64)
    want = (P @ gy).T @ (P @ x) / n
    assert _rel(tr.g_w, want) < 0.02


def test_reference_cuda_rounding_is_biased():
    """The reference op's mantissa-driven rounding (kept for characterisation
    only): values with an all-zero mantissa (0 and the powers of two) are
    rounded UP, so it cannot be unbiased."""
    assert orc.stoch_round_mantissa(np.array([2.0, -3.0, 0.0, 4.0], F32)).tolist() == [3, -3, 1, 5]


# ------------------------------------------------------------------ frozen snapshots of the oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("name", ["nearest_int4_L320_O64_I48", "stoch_row_int8_L192_O32_I40"])
def test_oracle_matches_its_frozen_snapshots(name):
    """tests/golden/*.npz were written by tests/golden/make_fixtures.py from this oracle: any change of
    its arithmetic (butterfly order, rounding, RNG numbering, nibble order) shows up here."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    data_seed, L, O, I, kw = mk.CASES[name]
    fresh = mk.case(data_seed, L, O, I, **kw)
    frozen = np.load(os.path.join(GOLDEN, name + ".npz"))
    assert set(frozen.files) == set(fresh)
    for k in frozen.files:
        assert np.array_equal(frozen[k], np.asarray(fresh[k])), k


# ------------------------------------------------------------------ 3-D activations (per-sample steps)

def test_batched_oracle_reduces_to_the_2d_path():
    """One sample: the batched functions are the 2-D ones, stochastic rounding included (the element
    numbering coincides).  Several samples under round-to-nearest: every sample is an independent 2-D
    problem with steps of its own, g_x stacks and g_W adds (n is a power of two, so dividing each
    sample's gradient by n or the sum gives the same fp32 numbers)."""
    rng = np.random.default_rng(3)
    B, T, O, I = 3, 32, 48, 24
    x = rng.standard_normal((B, T, I)).astype(np.float32)
    w = rng.standard_normal((O, I)).astype(np.float32) * 0.1
    gy = (rng.standard_normal((B, T, O)) * np.array([1e-3, 5e-2, 2.0])[:, None, None]).astype(np.float32)
    n, rows = orc.hla_rows(T)
    assert n == 32
    for kw in (dict(), dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW), dict(act_scale=orc.SCALE_SAWB, w_scale=orc.SCALE_SAWB)):
        cfg = orc.HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows), **kw)
        xq, sx = orc.abc_forward_batched(x, cfg)
        gx, gw, traces = orc.linear_backward_batched(gy, w, xq, sx, cfg)
        acc = np.zeros((O, I), dtype=np.float32)
        for b in range(B):
            xq_b, sx_b = orc.abc_forward(x[b], cfg)
            assert np.array_equal(xq[b], xq_b) and sx[b] == sx_b[0]
            tr = orc.linear_backward(gy[b], w, xq_b, sx_b, cfg)
            assert np.array_equal(gx[b], tr.g_x)
            assert np.array_equal(traces[b].qG, tr.qG) and np.array_equal(traces[b].qGp, tr.qGp)
            acc = (acc + tr.g_w).astype(np.float32)
        assert np.array_equal(gw, acc)
        # the three samples differ by orders of magnitude: shared steps would crush the small ones
        assert len({float(s) for s in sx}) == B and traces[0].sG.max() < traces[2].sG.min()
    # the order of the sum over samples: ranges of ceil(B / ranges) samples, then the range sums
    B5 = 5
    x5 = rng.standard_normal((B5, T, I)).astype(np.float32)
    gy5 = (rng.standard_normal((B5, T, O)) * (10.0 ** rng.uniform(-3, 1, (B5, 1, 1)))).astype(np.float32)
    cfg = orc.HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows))
    xq5, sx5 = orc.abc_forward_batched(x5, cfg)
    per_sample = [orc.linear_backward(gy5[b], w, *orc.abc_forward(x5[b], cfg), cfg).g_w for b in range(B5)]
    f32 = np.float32
    seq = per_sample[0]
    for p in per_sample[1:]:
        seq = (seq + p).astype(f32)
    two = (((per_sample[0] + per_sample[1]).astype(f32) + per_sample[2]).astype(f32)
           + (per_sample[3] + per_sample[4]).astype(f32)).astype(f32)
    assert np.array_equal(orc.linear_backward_batched(gy5, w, xq5, sx5, cfg)[1], seq)
    assert np.array_equal(orc.linear_backward_batched(gy5, w, xq5, sx5, cfg, gw_ranges=2)[1], two)
    assert not np.array_equal(seq, two)                 # the order is visible in the last bits
    assert np.array_equal(orc.linear_backward_batched(gy5, w, xq5, sx5, cfg, gw_ranges=5)[1], seq)   # one sample per range

    cfg = orc.HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows), gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH,
                        act_round=orc.ROUND_STOCH, seed=77)
    xq1, sx1 = orc.abc_forward_batched(x[:1], cfg)
    xq2, sx2 = orc.abc_forward(x[0], cfg)
    assert np.array_equal(xq1[0], xq2) and sx1[0] == sx2[0]
    gx1, gw1, _ = orc.linear_backward_batched(gy[:1], w, xq1, sx1, cfg)
    tr = orc.linear_backward(gy[0], w, xq2, sx2, cfg)
    assert np.array_equal(gx1[0], tr.g_x) and np.array_equal(gw1, tr.g_w)


# ------------------------------------------------------------------ low-rank g_x schemes

def test_hla_expand_is_the_transposed_projection():
    """P^T t against the explicit block-diagonal matrix product (integer inputs: exact), P P^T = n I
    (projecting the expansion gives n times the coefficients back), and the full-rank round trip."""
    rng = np.random.default_rng(5)
    for n, rows in (orc.hla_rows(64), orc.paper_rows(16, 8), orc.hla_rows(8), (1, np.array([0]))):
        r, nb, C = len(rows), 3, 7
        t = rng.integers(-40, 40, (nb * r, C)).astype(np.float32)
        P = orc.hadamard(n).astype(np.float64)[np.asarray(rows)]
        ref = np.concatenate([P.T @ t[b * r:(b + 1) * r].astype(np.float64) for b in range(nb)])
        out = orc.hla_expand(t, n, rows)
        assert out.dtype == np.float32 and np.array_equal(out, ref.astype(np.float32))
        assert np.array_equal(orc.fwht_blocks_first(out, n, np.asarray(rows)), n * t)
    x = rng.standard_normal((128, 3)).astype(np.float32)
    full = np.arange(32)
    assert np.abs(orc.hla_expand(orc.fwht_blocks_first(x, 32, full), 32, full) / 32 - x).max() < 1e-5


def test_gx_lowrank_against_the_port_and_the_plain_product():
    """The oracle's g_x of the schemes low_rank / gilr_gwh: within tolerance of the op-for-op port of those
    branches, and, with INT8 codes and every coefficient kept, close to the plain product g_y W."""
    import torch
    from oracle import fakequant_port as fq
    L, O, I = 448, 64, 40
    torch.manual_seed(0)
    x, w, gy = torch.randn(L, I), torch.randn(O, I) * 0.1, torch.randn(L, O) * 1e-3
    n, rows = orc.hla_rows(L)
    cfg = orc.HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows))
    got = orc.gx_lowrank(gy.numpy(), w.numpy(), cfg).g_x
    P = torch.tensor(orc.make_WHT(L), dtype=torch.float32)
    xq, sx = fq.setup_context(x, P, fq.PortConfig())
    for scheme, h_out, h_bs in (("low_rank", torch.zeros(1, 1), P),
                                ("gilr_gwh", P, torch.tensor(orc.make_hadamard(L), dtype=torch.float32))):
        xq, sx = fq.setup_context(x, h_bs, fq.PortConfig())
        gi, _ = fq.backward(gy, w, xq, sx, h_out, h_bs, fq.PortConfig(), scheme=scheme)
        assert np.linalg.norm(got - gi.numpy()) / np.linalg.norm(gi.numpy()) < 1e-3
    full = orc.HotConfig(hla_n=16, hla_rows=tuple(range(16)), gx_bits=8, w_bits=8)
    exact = (gy @ w).numpy()
    assert np.linalg.norm(orc.gx_lowrank(gy.numpy(), w.numpy(), full).g_x - exact) / np.linalg.norm(exact) < 0.02
    # the projection loses what the dropped rows carried: g_x equals P^T P (g_y W) / n up to quantisation
    proj = orc.hla_expand(orc.fwht_blocks_first(exact.astype(np.float32), n, np.asarray(rows)), n, rows) / n
    hi = orc.HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows), gx_bits=8, w_bits=8)
    assert np.linalg.norm(orc.gx_lowrank(gy.numpy(), w.numpy(), hi).g_x - proj) / np.linalg.norm(proj) < 0.02


# ------------------------------------------------------------------ logarithmic quantiser

def test_luq_levels_step_and_expectation():
    """luq_quantizer_BWD (utils/quant_matmul.py:58-77): the step is max / 2^7, codes are 0 or +-2^j, the
    maximum maps to 2^7 exactly, a value between two levels lands on one of the two, and the mean over many
    seeds converges on the value: both for the underflow region (|t| < s: s with probability |t| / s) and for
    the logarithmic rounding (the larger level with probability m / 2^k - 1)."""
    rng = np.random.default_rng(1)
    t = (rng.standard_normal((48, 40)) * 2e-3).astype(np.float32)
    t[0, 0] = np.float32(9e-3)                               # the maximum
    t[0, 1:6] = np.float32(9e-3) * np.array([2.0 ** -9, 2.0 ** -8, 3 * 2.0 ** -7, 0.75, -0.6], dtype=np.float32)
    q, s = orc.luq_quant(t, 4, seed=0)
    assert s[0] == np.float32(9e-3) / np.float32(128) and q[0, 0] == 128
    mags = np.unique(np.abs(q))
    assert set(mags.tolist()) <= {0} | {2 ** j for j in range(11)}
    m = np.abs(t) / s[0]
    inside = (m >= 1) & (np.abs(t) <= t.max())
    k = np.floor(np.log2(m[inside])).astype(int)
    assert np.all((np.abs(q[inside]) == 2 ** k) | (np.abs(q[inside]) == 2 ** (k + 1)))
    assert np.array_equal(np.sign(q[q != 0]), np.sign(t[q != 0]))
    small = m < 1
    assert set(np.abs(q[small]).tolist()) <= {0, 1}
    N = 800
    acc = np.zeros(t.shape)
    for seed in range(N):
        acc += orc.luq_quant(t, 4, seed=seed)[0]
    mean = acc / N * s[0]
    ok = np.abs(t) <= t.max()
    # standard error of a two-point variable with gap <= 2^k s <= |t|: <= |t| / (2 sqrt N); five sigma
    assert np.all(np.abs(mean - t)[ok] <= 5 * np.maximum(np.abs(t), s[0])[ok] / (2 * np.sqrt(N)) + 1e-12)
    # exact levels stay where they are; zero stays zero; a tensor without a positive element gives zeros
    lv = (np.array([[1, 2, 4, 64, 128, 0, -8]], dtype=np.float32) * np.float32(2.0 ** -10))
    q2, s2 = orc.luq_quant(lv, 4, seed=3)
    assert s2[0] == np.float32(2.0 ** -10) and np.array_equal(q2, [[1, 2, 4, 64, 128, 0, -8]])
    q3, s3 = orc.luq_quant(-np.abs(t), 4, seed=0)
    assert not q3.any() and s3[0] <= 0


def test_luq_saturation_of_the_product_form():
    """The reference's logarithmic codes have no upper bound (the step is max(t) / 2^7, not absmax / 2^7:
    utils/quant_matmul.py:60-61,71-74); the two-plane INT8 product saturates at 2^10.  The bound changes
    a code only for negative elements of at least eight times the positive maximum, and then to -2^10."""
    t = np.array([[1e-3, -0.5, 2e-4, -3e-2, -7.9e-3, 5e-4]], dtype=np.float32)
    free, s = orc.luq_quant(t, 4, seed=0)
    held, s2 = orc.luq_quant(t, 4, seed=0, max_exp=orc.LUQ_PRODUCT_MAX_EXP)
    assert s[0] == s2[0] == np.float32(1e-3) / np.float32(128)
    assert free[0, 1] in (-32768, -65536) and free[0, 3] in (-2048, -4096)       # 500 x and 30 x the maximum
    assert held[0, 1] == -1024 and held[0, 3] == -1024
    below = np.abs(t[0]) < 1024 * s[0]
    assert np.array_equal(free[0, below], held[0, below]) and below.tolist() == [True, False, True, False, True, True]
    # -7.9e-3 is 1011 s: its code may round up to 1024 but not beyond; held and free agree whenever free <= 1024
    assert abs(int(held[0, 4])) in (512, 1024) and (free[0, 4] == held[0, 4])
    rng = np.random.default_rng(5)
    for seed in range(20):
        u = (rng.standard_normal((16, 32)) * 1e-3).astype(np.float32)
        a, _ = orc.luq_quant(u, 4, seed=seed)
        b, _ = orc.luq_quant(u, 4, seed=seed, max_exp=10)
        assert np.array_equal(np.clip(a, -1024, 1024), b)
        if np.abs(u).max() < 8 * u.max():
            assert np.array_equal(a, b)
    # gx_luq is the product form: saturated by default, the reference's codes on request
    gy = (rng.standard_normal((32, 32)) * 1e-3).astype(np.float32)
    gy[3, :16] = -0.4                                  # one block whose transform is far below -max
    w = (rng.standard_normal((32, 24)) * 0.1).astype(np.float32)
    tr_h, tr_f = orc.gx_luq(gy, w, orc.HotConfig(seed=1)), orc.gx_luq(gy, w, orc.HotConfig(seed=1), max_exp=None)
    assert np.abs(tr_h.qG).max() == 1024 and np.abs(tr_f.qG).max() > 1024
    keep = np.ones(32, bool); keep[3] = False
    assert np.array_equal(tr_h.g_x[keep], tr_f.g_x[keep])


def test_gw_luq_mean_is_the_product_with_the_dequantised_buffer():
    """gw_luq = (luq((P g_y)^T) . xq^T) s s_x / n: the quantiser is unbiased, so the mean over seeds
    converges on ((P g_y)^T . (xq s_x)^T) / n, a plain float product of the projection (computed here from
    the explicit matrix P, not from the butterflies) with the dequantised buffer.  A transposed operand,
    a dropped step or the wrong divisor misses it by far more than the sampling error; the rows are
    padded (L' = 21 -> 24), which moves the element numbers only."""
    rng = np.random.default_rng(8)
    L, O, I = 56, 24, 16
    gy = (rng.standard_normal((L, O)) * 1e-3).astype(np.float32)
    x = rng.standard_normal((L, I)).astype(np.float32)
    n, rows = orc.hla_rows(L)
    lp = (L // n) * len(rows)
    assert (n, lp) == (8, 21)
    cfg = orc.HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows), gw_bits=4)
    xq, sx = orc.abc_forward(x, cfg)
    P = np.kron(np.eye(L // n), orc.make_WHT(n).astype(np.float64))                    # [L', L]
    target = (P @ gy.astype(np.float64)).T @ (xq.astype(np.float64) * float(sx[0])) / n
    N = 300
    acc = np.zeros_like(target)
    for seed in range(N):
        acc += orc.gw_luq(gy, xq, sx, replace(cfg, seed=seed))
    assert np.linalg.norm(acc / N - target) / np.linalg.norm(target) < 0.05
    one = orc.gw_luq(gy, xq, sx, cfg)
    assert one.shape == (O, I) and one.dtype == np.float32
    assert np.linalg.norm(one - target) / np.linalg.norm(target) > 0.05                # a single draw is coarse
    # element numbering: padded rows, stream 5 -- a different stream or the unpadded numbering draws other codes
    Gt = np.ascontiguousarray(orc.fwht_blocks_first(gy, n, np.asarray(rows)).T)
    idx = np.arange(O)[:, None] * 24 + np.arange(lp)[None, :]
    q, s = orc.luq_quant(Gt, 4, 0, stream=orc.STREAM_LUQ_GW, index=idx, max_exp=10)
    ref = ((orc.int_gemm_nt(q, xq.T).astype(np.float32) * s[0]) * sx[0]) / np.float32(n)
    assert np.array_equal(orc.gw_luq(gy, xq, sx, replace(cfg, seed=0)), ref.astype(np.float32))


def test_gx_luq_close_to_the_plain_product():
    rng = np.random.default_rng(2)
    L, O, I = 256, 64, 48
    gy = (rng.standard_normal((L, O)) * 1e-3).astype(np.float32)
    w = (rng.standard_normal((O, I)) * 0.1).astype(np.float32)
    exact = gy @ w
    acc = np.zeros_like(exact, dtype=np.float64)
    for seed in range(40):
        acc += orc.gx_luq(gy, w, orc.HotConfig(seed=seed)).g_x
    # unbiased in g_y; what remains is the 4-bit weight quantiser
    wq, sw = orc.quant(orc.fwht_blocks_first(w, 16), 4)
    w_hat = orc.fwht_blocks_first((wq * sw[0]).astype(np.float32), 16) / 16
    target = gy @ w_hat
    assert np.linalg.norm(acc / 40 - target) / np.linalg.norm(target) < 0.08
