"""Canonical CPU oracle (NumPy, fp32) for the HOT linear backward path.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Every function restates one piece of the reference's fake-quant path
(/root/reference/utils/quant_matmul.py, utils/hadamard_matmul.py) or of the
wire format of its CUDA op (cuda_measure/HLQ_backward_kernel.cu); the cited
file:line is given per function.  Two deliberate, documented differences:

* Transforms are evaluated as fp32 butterflies in ONE fixed order
  (h = 1, 2, 4, ...; (x+y, x-y)), the order of the reference CUDA kernel
  ``fwht_kernel`` (HLQ_backward_kernel.cu:63-78), instead of the BLAS matmul
  ``reshape(-1, n) @ H`` of hadamard_matmul.py:121-161 whose last-ulp
  summation order depends on the BLAS build.  Mathematically identical.
* Stochastic rounding draws 16-bit uniforms from Philox-4x32-7 keyed by
  (seed, element index) instead of the global torch generator
  (quant_matmul.py:96) and rounds in 16.16 fixed point (sr_codes), so that CPU
  and GPU agree bit for bit.

How each function is pinned (tests/test_oracle_*.py):
  pow2_factor / pow2_factor_max16   closed form n & -n; hand-derived table
  hadamard                          scipy.linalg.hadamard; H H^T = n I
  sequency_of_natural / wht_rows    brute-force sign-change count + stable sort
  kept_sequencies                   hand-derived sets for n = 1, 2, 4, 16, 64
  fwht_blocks_last / _first         explicit block-diagonal matmul on small
                                    integer inputs (exact in fp32)
  quant_rne / quant_sr / quant_sawb textbook absmax quantiser; ties-to-even
                                    table; all-zero input; max -> +-qmax;
                                    SR mean/variance; Philox known answers
  pack_int4 / unpack_int4           all 225 code pairs round trip; byte value
                                    formula of HLQ_backward_kernel.cu:140
  int_gemm_nt                       numpy int64 matmul
  linear_backward / abc_forward     composition; with quantisation off and
                                    r = n they equal g_y W and g_y^T x
No function here is "parity unpinned" except the last-ulp BLAS summation order
of the reference's transform matmuls, which is intentionally not matched.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import numpy as np

F32 = np.float32
EPS = 1e-11  # args.py:34

# --------------------------------------------------------------------------
# sizes and matrices
# --------------------------------------------------------------------------


def pow2_factor(size: int) -> int:
    """Largest power-of-two divisor of ``size`` (hadamard_matmul.py:9-15)."""
    if size < 1:
        raise ValueError("size must be >= 1")
    return size & -size


def pow2_factor_max16(size: int) -> int:
    """hadamard_matmul.py:17-27: as pow2_factor but 16 when the factor exceeds
    16 (and size > 16)."""
    p = pow2_factor(size)
    return 16 if (p > 16 and size > 16) else p


def hadamard(n: int) -> np.ndarray:
    """Sylvester Hadamard matrix, natural order, entries +-1
    (hadamard_matmul.py:32-51).  H[i, j] = (-1)^popcount(i & j)."""
    if n < 1 or (n & (n - 1)):
        raise ValueError("n must be int and power of 2.")
    i = np.arange(n, dtype=np.int64)
    a = i[:, None] & i[None, :]
    pc = np.zeros_like(a)
    while a.any():
        pc += a & 1
        a >>= 1
    return (1 - 2 * (pc & 1)).astype(np.int64)


def make_hadamard(size: int) -> np.ndarray:
    """hadamard_matmul.py:57-59."""
    return hadamard(pow2_factor_max16(size))


def sequency_of_natural(n: int) -> np.ndarray:
    """seq[i] = number of sign changes along row i of the Sylvester matrix
    = gray_decode(bit_reverse(i)).  (Replaces the row sort by counted sign
    changes of hadamard_matmul.py:210-213.)"""
    bits = n.bit_length() - 1
    out = np.zeros(n, dtype=np.int64)
    for i in range(n):
        r = 0
        for b in range(bits):
            if i >> b & 1:
                r |= 1 << (bits - 1 - b)
        g = r
        s = r >> 1
        while s:
            g ^= s
            s >>= 1
        out[i] = g
    return out


def natural_of_sequency(n: int) -> np.ndarray:
    """Inverse permutation of sequency_of_natural."""
    seq = sequency_of_natural(n)
    inv = np.empty(n, dtype=np.int64)
    inv[seq] = np.arange(n)
    return inv


def kept_sequencies(n: int, percentile: float = 50) -> np.ndarray:
    """Sequency indices kept by the low-rank selection of make_WHT
    (hadamard_matmul.py:215-225), increasing order."""
    # biggest_sqrt_factor (hadamard_matmul.py:172-178): largest power of 4 <= n
    p4 = 1
    while p4 * 4 <= n:
        p4 *= 4
    s = int(math.isqrt(p4))
    sf = int(0.1 * (-np.sqrt(2 * s ** 2 * percentile + 25) + 10 * s + 5))
    idx = np.arange(n)
    parts = []
    for i in range(s):
        if i % 2 == 0:
            parts.append(idx[s * i: s * (i + 1) - (i + sf)])
        else:
            parts.append(idx[s * i + (i + sf): s * (i + 1)])
    return np.concatenate(parts).astype(np.int64)


def hla_rows(size: int, percentile: float = 50) -> Tuple[int, np.ndarray]:
    """(n, natural-order row index of each kept coefficient, in output order)
    for a token count ``size``: the python rule of make_WHT
    (hadamard_matmul.py:209-226; n = make_non_block_hadamard :167-170)."""
    n = 1 if size == 1 else pow2_factor(size)
    keep = kept_sequencies(n, percentile)
    return n, natural_of_sequency(n)[keep]


def make_WHT(size: int, percentile: float = 50) -> np.ndarray:
    """The r x n matrix P of hadamard_matmul.py:209-226."""
    n, rows = hla_rows(size, percentile)
    return hadamard(n)[rows]


def paper_rows(n: int = 16, r: int = 8) -> Tuple[int, np.ndarray]:
    """Cost-model setting (analysis_calculator.py:174-175): the r lowest
    sequencies of an n-block."""
    return n, natural_of_sequency(n)[np.arange(r)]


# --------------------------------------------------------------------------
# transforms, canonical butterfly order (HLQ_backward_kernel.cu:63-78)
# --------------------------------------------------------------------------


def _fwht_axis(v: np.ndarray, axis: int) -> np.ndarray:
    """Unnormalised FWHT of length v.shape[axis] (a power of two) along
    ``axis``: stages h = 1, 2, 4, ...; pair (j, j+h) with (j // h) even becomes
    (v[j] + v[j+h], v[j] - v[j+h]).  fp32 throughout."""
    v = np.ascontiguousarray(np.moveaxis(v, axis, -1), dtype=F32).copy()
    n = v.shape[-1]
    h = 1
    while h < n:
        w = v.reshape(v.shape[:-1] + (n // (2 * h), 2, h))
        a = w[..., 0, :].copy()
        b = w[..., 1, :].copy()
        w[..., 0, :] = a + b
        w[..., 1, :] = a - b
        h *= 2
    return np.moveaxis(v, -1, axis)


def fwht_blocks_last(a: np.ndarray, n: int) -> np.ndarray:
    """A [.., K] -> each contiguous n-chunk of the last dim times H_n:
    lowering_matmul_front(A, H_n) (hadamard_matmul.py:121-141)."""
    a = np.asarray(a, dtype=F32)
    k = a.shape[-1]
    if k % n:
        raise ValueError("last dim must be a multiple of n")
    return _fwht_axis(a.reshape(a.shape[:-1] + (k // n, n)), -1).reshape(a.shape)


def fwht_blocks_first(a: np.ndarray, n: int, rows: Optional[np.ndarray] = None) -> np.ndarray:
    """A [R, C] -> H_n applied to every block of n consecutive rows; when
    ``rows`` (natural-order indices) is given only those coefficients of each
    block are kept, in that order: out[b*r + k, :] = T_b[rows[k], :].
    = lowering_matmul_back(H_n or P, A) (hadamard_matmul.py:143-161)."""
    a = np.asarray(a, dtype=F32)
    R, C = a.shape
    if R % n:
        raise ValueError("row count must be a multiple of n")
    t = _fwht_axis(a.reshape(R // n, n, C), 1)
    if rows is not None:
        t = t[:, np.asarray(rows), :]
    return np.ascontiguousarray(t.reshape(-1, C))


# --------------------------------------------------------------------------
# Philox-4x32-10 (Salmon et al., SC'11) -- counter-based uniforms for SR
# --------------------------------------------------------------------------

_PH_M0 = np.uint64(0xD2511F53)
_PH_M1 = np.uint64(0xCD9E8D57)
_PH_W0 = 0x9E3779B9
_PH_W1 = 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32(c0, c1, c2, c3, k0: int, k1: int, rounds: int = 10):
    """Vectorised Philox-4x32; counters are uint32 arrays, key two ints."""
    c0 = np.asarray(c0, dtype=np.uint64)
    c1 = np.asarray(c1, dtype=np.uint64)
    c2 = np.asarray(c2, dtype=np.uint64)
    c3 = np.asarray(c3, dtype=np.uint64)
    k0 &= 0xFFFFFFFF
    k1 &= 0xFFFFFFFF
    for _ in range(rounds):
        p0 = _PH_M0 * c0
        p1 = _PH_M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & _MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & _MASK
        c0, c1, c2, c3 = (hi1 ^ c1 ^ np.uint64(k0)), lo1, (hi0 ^ c3 ^ np.uint64(k1)), lo0
        k0 = (k0 + _PH_W0) & 0xFFFFFFFF
        k1 = (k1 + _PH_W1) & 0xFFFFFFFF
    return (c0.astype(np.uint32), c1.astype(np.uint32), c2.astype(np.uint32), c3.astype(np.uint32))


SR_PHILOX_ROUNDS = 7   # Philox-4x32-7: the fewest rounds Random123 reports as passing BigCrush (10 is its default margin)


def sr_bits16(index: np.ndarray, seed: int, stream: int) -> np.ndarray:
    """A 16-bit uniform integer (uint32 array) for the element with linear index
    ``index`` (int64 array).  One Philox-4x32-7 call serves eight consecutive
    elements: counter = (index>>3 lo, index>>3 hi, stream, 0), key = (seed lo,
    seed hi); element index & 7 = 2 i + h takes the low (h = 0) or high (h = 1)
    16 bits of output word i.  The 10-round function is pinned by Random123's
    known answers; seven rounds are the same round function and key schedule
    applied seven times."""
    index = np.asarray(index, dtype=np.uint64)
    q = index >> np.uint64(3)
    w = philox4x32(q & _MASK, q >> np.uint64(32), np.full(q.shape, stream, np.uint64),
                   np.zeros(q.shape, np.uint64), seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF, rounds=SR_PHILOX_ROUNDS)
    slot = (index & np.uint64(7)).astype(np.int64)
    word = np.choose(slot >> 1, w).astype(np.uint32)
    return np.where((slot & 1) == 0, word & np.uint32(0xFFFF), word >> np.uint32(16)).astype(np.uint32)


def sr_uniform(index: np.ndarray, seed: int, stream: int) -> np.ndarray:
    """u in [0, 1) on a 2^-16 grid: sr_bits16 * 2^-16 (the logarithmic quantiser's two uniforms)."""
    return (sr_bits16(index, seed, stream).astype(F32) * F32(2.0 ** -16)).astype(F32)


def sr_codes(t: np.ndarray, d: np.ndarray, qmax: int, index: np.ndarray, seed: int, stream: int) -> np.ndarray:
    """Stochastic rounding of t / d to integers of magnitude <= qmax, in the fixed-point form the
    kernels use: with rcp = fl32(1 / d),
        p = fl32(|t| * (rcp * 2^16) + 0.5)        one fused multiply-add: |t| / d in units of 2^-16, rounded
        q = sign(t) * min((trunc(p) + r) >> 16, qmax),   r = sr_bits16(element)
    i.e. floor(|y|) + 1 with probability frac(|y|) taken on a 2^-16 grid, y = t / d: the stochastic
    rounding of stoch_quantizer_BWD / norm_quantizer_BWD (utils/quant_matmul.py:19-31, 86-100) with a
    counter-based generator.  The product with the reciprocal stands for the division (at most 1.5 ulp
    apart) and the grid rounds the probability to the nearest 2^-16: E[q] is within 2^-15 of y."""
    return sr_round(t, d, qmax, sr_bits16(index, seed, stream))


def sr_round(t: np.ndarray, d: np.ndarray, qmax: int, r: np.ndarray) -> np.ndarray:
    """The arithmetic of sr_codes for given 16-bit integers r."""
    t = np.asarray(t, dtype=F32)
    rcpk = ((F32(1.0) / np.asarray(d, dtype=F32)).astype(F32) * F32(65536.0)).astype(F32)
    # fused multiply-add in fp32 = the exact product and sum, rounded once.  The product of two fp32
    # numbers is exact in float64, and so is the sum with 0.5 wherever it can reach 1 (48 significant
    # bits from 2^-1 up); below that the truncation gives 0 whatever the last bit
    p = (np.abs(t).astype(np.float64) * rcpk.astype(np.float64) + 0.5).astype(F32)
    m = np.minimum((np.trunc(p).astype(np.int64) + np.asarray(r).astype(np.int64)) >> 16, qmax)
    return np.where(t < 0, -m, m)


# --------------------------------------------------------------------------
# quantisers
# --------------------------------------------------------------------------

ROUND_NEAREST = 0
ROUND_STOCH = 1
SCALE_TENSOR = 0
SCALE_ROW = 1
SCALE_SAWB = 2

STREAM_GX = 0   # g_y H  quantiser
STREAM_GW = 1   # (P g_y)^T quantiser
STREAM_W = 2    # H W quantiser
STREAM_ACT = 3  # P x quantiser


def _qmax(bits: int) -> int:
    return 2 ** (bits - 1) - 1


def quant_scale(t: np.ndarray, bits: int, mode: int) -> np.ndarray:
    """Step size s (WITHOUT eps) and clip: int_quantizer_BWD
    (quant_matmul.py:112-113), norm_quantizer_BWD (:20-21),
    sawb_quantizer_BWD (:41-44).  Returns (s, clip) broadcastable to t."""
    t = np.asarray(t, dtype=F32)
    q = F32(_qmax(bits))
    if mode == SCALE_TENSOR:
        mx = np.max(np.abs(t)).astype(F32) if t.size else F32(0)
        return (mx / q).astype(F32), mx
    if mode == SCALE_ROW:
        mx = np.max(np.abs(t), axis=1, keepdims=True).astype(F32)
        return (mx / q).astype(F32), mx
    if mode == SCALE_SAWB:
        # sums in float64, result rounded to fp32 once
        t64 = t.astype(np.float64)
        clip = F32(12.1 * np.sqrt(np.mean(t64 * t64)) - 12.2 * np.mean(np.abs(t64)))
        return (clip / q).astype(F32), clip
    raise ValueError("bad scale mode")


def quant(t: np.ndarray, bits: int, mode: int = SCALE_TENSOR, rounding: int = ROUND_NEAREST,
          seed: int = 0, stream: int = 0, index: Optional[np.ndarray] = None):
    """Codes (int8) and step size s (fp32, without eps).

    y = clamp(t, -clip, clip) / fl32(s + 1e-11)           (IEEE fp32 division)
    nearest:     q = rint(y), ties to even   (int_quantizer_BWD  :112-116,
                                              sawb_quantizer_BWD :40-49)
    stochastic:  q = sign(y) (floor|y| + Bernoulli(|y| - floor|y|)), evaluated by sr_codes
                                             (stoch_quantizer_BWD :86-100,
                                              norm_quantizer_BWD  :19-31)
    ``index`` gives the RNG element index of every entry (default: row-major
    position in t)."""
    t = np.asarray(t, dtype=F32)
    s, clip = quant_scale(t, bits, mode)
    d = (s + F32(EPS)).astype(F32)
    y = (np.clip(t, -clip, clip).astype(F32) / d).astype(F32)
    if rounding == ROUND_NEAREST:
        q = np.rint(y)
    else:
        if index is None:
            index = np.arange(t.size, dtype=np.int64).reshape(t.shape)
        q = sr_codes(np.clip(t, -clip, clip).astype(F32), d, _qmax(bits), index, seed, stream)
    qm = _qmax(bits)
    q = np.clip(q, -qm, qm)  # never active for absmax scales; guards sawb/eps
    s_out = s.reshape(-1) if mode == SCALE_ROW else np.asarray(s, dtype=F32).reshape(1)
    return q.astype(np.int8), s_out.astype(F32)


# --------------------------------------------------------------------------
# INT4 wire format (HLQ_backward_kernel.cu:135-140; = cutlass::int4b_t order)
# --------------------------------------------------------------------------


def pack_int4(q: np.ndarray) -> np.ndarray:
    """[.., K] int8 codes in [-8, 7] -> [.., K/2] bytes; byte j holds element
    2j in bits 3:0 and element 2j+1 in bits 7:4 (two's complement nibbles)."""
    q = np.asarray(q, dtype=np.int8)
    if q.shape[-1] % 2:
        raise ValueError("K must be even")
    u = q.view(np.uint8)
    return ((u[..., 1::2] << 4) | (u[..., 0::2] & 0x0F)).astype(np.uint8).view(np.int8)


def unpack_int4(p: np.ndarray) -> np.ndarray:
    p = np.asarray(p).view(np.uint8)
    lo = (p & 0x0F).astype(np.int16)
    hi = (p >> 4).astype(np.int16)
    lo = np.where(lo > 7, lo - 16, lo)
    hi = np.where(hi > 7, hi - 16, hi)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.int8)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    return out


# --------------------------------------------------------------------------
# integer GEMM contract (HLQ_backward_kernel.cu:181-280, 309-384)
# --------------------------------------------------------------------------


def int_gemm_nt(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """C[M, N] (int32) = A[M, K] . B[N, K]^T on integer codes.  Evaluated in
    float64 BLAS, exact because |acc| <= 127^2 K << 2^53."""
    c = np.asarray(a, dtype=np.float64) @ np.asarray(b, dtype=np.float64).T
    return np.rint(c).astype(np.int64).astype(np.int32)


# --------------------------------------------------------------------------
# the path: forward activation buffer (ABC) and backward
# --------------------------------------------------------------------------


@dataclass
class HotConfig:
    """The knobs FLinearQ reads from the module ``args`` (args.py:29-49),
    restricted to scheme ``gih_gwlr``."""
    n_o: int = 16                      # Hadamard block along O (make_hadamard)
    hla_n: int = 1                     # HLA block along tokens
    hla_rows: Sequence[int] = (0,)     # kept natural-order rows, output order
    gx_bits: int = 4                   # GogiQuantBit
    w_bits: int = 4                    # weightQuantBit
    gw_bits: int = 8                   # GogwQuantBit
    act_bits: int = 8                  # actQuantBit
    gx_round: int = ROUND_NEAREST      # quantBWDGogi: int | stoch | nq
    gx_scale: int = SCALE_TENSOR       #   nq = stochastic + SCALE_ROW
    w_round: int = ROUND_NEAREST       # quantBWDWgt: int | stoch | sawb
    w_scale: int = SCALE_TENSOR
    gw_round: int = ROUND_NEAREST      # quantBWDGogw
    gw_scale: int = SCALE_TENSOR
    act_round: int = ROUND_NEAREST     # quantBWDAct
    act_scale: int = SCALE_TENSOR
    seed: int = 0

    @staticmethod
    def python_rule(L: int, **kw) -> "HotConfig":
        n, rows = hla_rows(L)
        return HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows), **kw)

    @staticmethod
    def paper(n: int = 16, r: int = 8, **kw) -> "HotConfig":
        n, rows = paper_rows(n, r)
        return HotConfig(hla_n=n, hla_rows=tuple(int(v) for v in rows), **kw)


def abc_forward(x: np.ndarray, cfg: HotConfig):
    """FLinearQ.setup_context (quant_matmul.py:178-212), scheme gih_gwlr:
    x <- P x (HLA along tokens) then quantise to INT8.
    Returns (xq int8 [L', I], sx fp32 [1])."""
    xp = fwht_blocks_first(np.asarray(x, dtype=F32), cfg.hla_n, np.asarray(cfg.hla_rows))
    idx = colwise_rng_index(xp.shape[1], xp.shape[0] // len(cfg.hla_rows), cfg.hla_rows).T
    return quant(xp, cfg.act_bits, cfg.act_scale, cfg.act_round, cfg.seed, STREAM_ACT, index=idx)


def colwise_rng_index(C: int, NB: int, rows) -> np.ndarray:
    """RNG element index of every coefficient of a column-wise transformed
    matrix, laid out [C, NB * r] (K-major).  The kernels walk the kept
    coefficients of a block in increasing natural-row order and number them
    ((c * NB + block) * rpad + visit) with rpad = r rounded up to 8, so that one
    Philox call serves eight consecutive visits of a channel.  Blocks with a single kept
    coefficient (r = 1: the one-token blocks of token counts no power of two divides) are numbered
    c * NB + block (rpad = 1), so that eight consecutive blocks of a channel share a call."""
    rows = np.asarray(rows)
    r = len(rows)
    rpad = 1 if r == 1 else (r + 7) // 8 * 8
    visit = np.argsort(np.argsort(rows))                      # rank of rows[k] among the kept rows
    c = np.arange(C, dtype=np.int64)[:, None, None]
    b = np.arange(NB, dtype=np.int64)[None, :, None]
    return ((c * NB + b) * rpad + visit[None, None, :].astype(np.int64)).reshape(C, NB * r)


@dataclass
class BackwardTrace:
    qG: np.ndarray = None
    sG: np.ndarray = None
    qW: np.ndarray = None
    sW: np.ndarray = None
    acc_x: np.ndarray = None
    qGp: np.ndarray = None
    sGp: np.ndarray = None
    acc_w: np.ndarray = None
    g_x: np.ndarray = None
    g_w: np.ndarray = None


def linear_backward(g_y: np.ndarray, w: np.ndarray, xq: np.ndarray, sx: np.ndarray,
                    cfg: HotConfig) -> BackwardTrace:
    """FLinearQ.backward (quant_matmul.py:215-348), scheme gih_gwlr, 2-D inputs.

    g_y [L, O], w [O, I], xq int8 [L', I] with step sx (from abc_forward)."""
    g_y = np.asarray(g_y, dtype=F32)
    w = np.asarray(w, dtype=F32)
    L, O = g_y.shape
    tr = BackwardTrace()
    # :238  g_y blkdiag(H)  ; :244-257 quantise
    G = fwht_blocks_last(g_y, cfg.n_o)
    tr.qG, tr.sG = quant(G, cfg.gx_bits, cfg.gx_scale, cfg.gx_round, cfg.seed, STREAM_GX)
    # :270  blkdiag(H) W ; :276-285 quantise
    Wh = fwht_blocks_first(w, cfg.n_o)
    tr.qW, tr.sW = quant(Wh, cfg.w_bits, cfg.w_scale, cfg.w_round, cfg.seed, STREAM_W,
                         index=colwise_rng_index(Wh.shape[1], Wh.shape[0] // cfg.n_o, np.arange(cfg.n_o)).T)
    # :288-290, :343
    tr.acc_x = int_gemm_nt(tr.qG, tr.qW.T)
    sg = tr.sG.reshape(-1, 1) if cfg.gx_scale == SCALE_ROW else tr.sG.reshape(1, 1)
    tr.g_x = (((tr.acc_x.astype(F32) * sg).astype(F32) * tr.sW[0]).astype(F32) / F32(cfg.n_o)).astype(F32)
    # :301 (P g_y)^T ; :307-320 quantise
    GpT = np.ascontiguousarray(fwht_blocks_first(g_y, cfg.hla_n, np.asarray(cfg.hla_rows)).T)
    tr.qGp, tr.sGp = quant(GpT, cfg.gw_bits, cfg.gw_scale, cfg.gw_round, cfg.seed, STREAM_GW,
                           index=colwise_rng_index(GpT.shape[0], GpT.shape[1] // len(cfg.hla_rows), cfg.hla_rows))
    # :322-324, :344
    tr.acc_w = int_gemm_nt(tr.qGp, np.asarray(xq).T)
    sgw = tr.sGp.reshape(-1, 1) if cfg.gw_scale == SCALE_ROW else tr.sGp.reshape(1, 1)
    tr.g_w = (((tr.acc_w.astype(F32) * sgw).astype(F32) * F32(np.asarray(sx).reshape(-1)[0])).astype(F32)
              / F32(cfg.hla_n)).astype(F32)
    return tr


def hla_expand(t: np.ndarray, n: int, rows) -> np.ndarray:
    """P^T t for the block-diagonal P of kept Walsh-Hadamard rows (lowering_matmul_back(h.mT, t),
    utils/hadamard_matmul.py:143-161 with utils/quant_matmul.py:334-337): t [NB r, C] -> [NB n, C].
    H is symmetric, so P^T c = H_n z with z the coefficients c put back at their natural rows and
    zeros elsewhere; evaluated with the canonical butterflies (adding an exact zero changes nothing)."""
    t = np.asarray(t, dtype=F32)
    rows = np.asarray(rows)
    r = len(rows)
    nb = t.shape[0] // r
    z = np.zeros((nb, n, t.shape[1]), dtype=F32)
    z[:, rows, :] = t.reshape(nb, r, t.shape[1])
    return fwht_blocks_first(z.reshape(nb * n, t.shape[1]), n)


def gx_lowrank(g_y: np.ndarray, w: np.ndarray, cfg: HotConfig) -> BackwardTrace:
    """grad_input of the schemes that project g_y to low rank along the TOKENS for the g_x product
    (utils/quant_matmul.py, transform_scheme "low_rank" and "gilr_gwh"): :229-233 g_y <- P g_y [L', O];
    :244-257 quantise (one step for the tensor); :263-266 W is NOT transformed; :276-285 quantise W;
    :288-290 (q(P g_y) q(W)) s_g s_w [L', I]; :334-337 P^T (.) / n.  cfg.hla_n / cfg.hla_rows describe P,
    cfg.gx_* the quantiser of P g_y, cfg.w_* that of W.  Element numbering of stochastic rounding: the
    column-wise one, P g_y as [O channels][NB blocks][r], W as blocks of one row."""
    g_y = np.asarray(g_y, dtype=F32)
    w = np.asarray(w, dtype=F32)
    L, O = g_y.shape
    rows = np.asarray(cfg.hla_rows)
    tr = BackwardTrace()
    Gp = fwht_blocks_first(g_y, cfg.hla_n, rows)                                        # [L', O]
    if cfg.gx_scale == SCALE_ROW:
        # a step per coefficient row (norm_quantizer on [L', O], :19-37): elements numbered row-major
        tr.qG, tr.sG = quant(Gp, cfg.gx_bits, SCALE_ROW, cfg.gx_round, cfg.seed, STREAM_GX)
    else:
        tr.qG, tr.sG = quant(Gp, cfg.gx_bits, SCALE_TENSOR, cfg.gx_round, cfg.seed, STREAM_GX,
                             index=colwise_rng_index(O, L // cfg.hla_n, rows).T)
    tr.qW, tr.sW = quant(w, cfg.w_bits, cfg.w_scale, cfg.w_round, cfg.seed, STREAM_W,
                         index=colwise_rng_index(w.shape[1], w.shape[0], np.arange(1)).T)
    tr.acc_x = int_gemm_nt(tr.qG, tr.qW.T)                                              # [L', I]
    sg = tr.sG[:, None] if cfg.gx_scale == SCALE_ROW else tr.sG[0]
    t = ((tr.acc_x.astype(F32) * sg).astype(F32) * tr.sW[0]).astype(F32)
    tr.g_x = (hla_expand(t, cfg.hla_n, rows) / F32(cfg.hla_n)).astype(F32)
    return tr


STREAM_LUQ = 4  # the two uniforms per element of the logarithmic quantiser


LUQ_PRODUCT_MAX_EXP = 10  # largest exponent j of a code +-2^j that the two-plane INT8 product carries


def luq_quant(t: np.ndarray, bits: int, seed: int, stream: int = STREAM_LUQ, index: Optional[np.ndarray] = None,
              max_exp: Optional[int] = None):
    """luq_quantizer_BWD (utils/quant_matmul.py:58-77): logarithmic unbiased quantisation.  With
    lev = 2^(bits-1) - 1 and s = max(t) / 2^lev (the maximum, not the largest magnitude, :60-61):
      * magnitudes below s become s with probability |t| / s, else 0 (:62-67: u1 ~ U[0, 1));
      * every other magnitude m s, 2^k <= m < 2^(k+1), becomes 2^k s or 2^(k+1) s, the larger with
        probability m / 2^k - 1 (:71-74: noise = 2^k (u2 - 1/2), 2^floor(log2((m + noise) 4 / 3)),
        never below 2^k), so that the expectation is t;
    Returns (codes in units of s: 0 or +-2^j as int32, s fp32 [1]).  floor(log2(.)) is taken from the
    binary exponent (torch's float log2 can round an argument just below a power of two up to it).
    A tensor without a positive element has s <= 0 in the reference; here all codes are 0 then.
    Element e draws u1, u2 = the uniforms 2 e and 2 e + 1 of `stream`.
    `max_exp` = None is the reference: since s comes from the maximum and not from the largest
    magnitude, a negative element beyond -max(t) takes a code as large as its size asks for.  With
    `max_exp` = J codes saturate at +-2^J, which changes a code only where |t| >= 2^J s (the code is
    at most 2^(k+1) with 2^k <= |t| / s), i.e. for negative elements of at least 2^(J - lev) times the
    positive maximum: the form gx_luq uses."""
    t = np.asarray(t, dtype=F32)
    lev = 2 ** (bits - 1) - 1
    mx = max(float(t.max()), 0.0) if t.size else 0.0
    s = F32(F32(mx) / F32(2.0 ** lev))
    idx = np.arange(t.size, dtype=np.int64).reshape(t.shape) if index is None else np.asarray(index, dtype=np.int64)
    u1 = sr_uniform(2 * idx, seed, stream)
    u2 = sr_uniform(2 * idx + 1, seed, stream)
    if s <= 0:
        return np.zeros(t.shape, dtype=np.int32), np.array([s], dtype=F32)
    ax = np.abs(t)
    zero = (ax < (s * u1).astype(F32)) | (t == 0)
    m = (np.where(ax < s, s, ax).astype(F32) / s).astype(F32)                   # >= 1
    k = np.frexp(m)[1].astype(np.int64) - 1                                      # floor(log2 m)
    noise = (np.ldexp(F32(1.0), k).astype(F32) * (u2 - F32(0.5)).astype(F32)).astype(F32)
    v = (((m + noise).astype(F32) * F32(4.0)).astype(F32) / F32(3.0)).astype(F32)
    j = np.maximum(np.frexp(v)[1].astype(np.int64) - 1, k)
    if max_exp is not None:
        j = np.minimum(j, max_exp)
    q = (np.sign(t).astype(np.int64) * (np.int64(1) << j)).astype(np.int64)
    q[zero] = 0
    return q.astype(np.int32), np.array([s], dtype=F32)


def gx_luq(g_y: np.ndarray, w: np.ndarray, cfg: HotConfig, max_exp: Optional[int] = LUQ_PRODUCT_MAX_EXP) -> BackwardTrace:
    """grad_input with quantBWDGogi = "luq" (utils/quant_matmul.py:238, 252-253, 270, 276-285, 288-290, 343):
    g_y blkdiag(H) through the logarithmic quantiser (cfg.gx_bits, one step for the tensor), blkdiag(H) W
    through cfg's weight quantiser, their integer product, the two steps, / n_o.
    STATED DEVIATION from the reference: the codes saturate at +-2^max_exp (default 10: what an INT8
    product of two code planes q = 16 a + b against [16 w | w] can carry; the reference multiplies in
    floating point and has no bound).  It is reached only by negative elements of g_y blkdiag(H) beyond
    eight times the tensor's positive maximum; max_exp = None gives the reference's unbounded codes."""
    g_y = np.asarray(g_y, dtype=F32)
    w = np.asarray(w, dtype=F32)
    tr = BackwardTrace()
    G = fwht_blocks_last(g_y, cfg.n_o)
    tr.qG, tr.sG = luq_quant(G, cfg.gx_bits, cfg.seed, max_exp=max_exp)
    Wh = fwht_blocks_first(w, cfg.n_o)
    tr.qW, tr.sW = quant(Wh, cfg.w_bits, cfg.w_scale, cfg.w_round, cfg.seed, STREAM_W,
                         index=colwise_rng_index(Wh.shape[1], Wh.shape[0] // cfg.n_o, np.arange(cfg.n_o)).T)
    tr.acc_x = int_gemm_nt(tr.qG, tr.qW.T)
    tr.g_x = (((tr.acc_x.astype(F32) * tr.sG[0]).astype(F32) * tr.sW[0]).astype(F32) / F32(cfg.n_o)).astype(F32)
    return tr


STREAM_LUQ_GW = 5  # the logarithmic quantiser on the projected g_y of the g_W product


def gw_luq(g_y: np.ndarray, xq: np.ndarray, sx: np.ndarray, cfg: HotConfig,
           max_exp: Optional[int] = LUQ_PRODUCT_MAX_EXP) -> np.ndarray:
    """grad_weight with the logarithmic quantiser on the projected g_y (quantBWDGogw = "luq", or
    luq_quantizer picked for a layer's g_W under quantAuto; utils/quant_matmul.py:296-301 g_y <- (P g_y)^T
    [O, L'], :307-314 luq_quantizer at cfg.gw_bits, :322-324 (q . xq) s s_x, :339-346 / n).  xq [L', I]
    and sx as abc_forward returns them.  Element e = o K8 + k of the projected tensor, K8 = L' rounded up
    to a multiple of 8 (the kernel's rows are padded with zeros, which draw code 0), takes the uniforms
    2 e and 2 e + 1 of stream STREAM_LUQ_GW.  Codes saturate at +-2^max_exp as in gx_luq."""
    g_y = np.asarray(g_y, dtype=F32)
    rows = np.asarray(cfg.hla_rows)
    Gt = np.ascontiguousarray(fwht_blocks_first(g_y, cfg.hla_n, rows).T)                  # [O, L']
    O, lp = Gt.shape
    k8 = -(-lp // 8) * 8
    index = np.arange(O, dtype=np.int64)[:, None] * k8 + np.arange(lp, dtype=np.int64)[None, :]
    q, s = luq_quant(Gt, cfg.gw_bits, cfg.seed, stream=STREAM_LUQ_GW, index=index, max_exp=max_exp)
    acc = int_gemm_nt(q, np.asarray(xq).T)
    return (((acc.astype(F32) * s[0]).astype(F32) * F32(np.asarray(sx).reshape(-1)[0])).astype(F32) / F32(cfg.hla_n)).astype(F32)


def stoch_round_mantissa(x: np.ndarray) -> np.ndarray:
    """The reference CUDA op's pseudo-stochastic rounding
    (HLQ_backward_kernel.cu:19-36), kept only to characterise its bias; the
    build does not use it."""
    x = np.asarray(x, dtype=F32)
    bits = x.view(np.uint32)
    mant = bits & np.uint32(0x007FFFFF)
    prob = mant >> np.uint32(11)
    rnd = mant & np.uint32(0x7FF)
    flip = (prob <= rnd).astype(np.int64)
    sign = np.where(x < 0, -1, 1)
    return sign * (np.floor(np.abs(x)).astype(np.int64) + flip)


# --------------------------------------------------------------------------
# 3-D activations [B, T, C]: one set of steps per sample
# --------------------------------------------------------------------------


def abc_forward_batched(x: np.ndarray, cfg: HotConfig):
    """FLinearQ.setup_context on a 3-D input (quant_matmul.py:178-212 with the vmapped quantisers
    :33-37,51-55,102-106,118-122 and the 3-D branch of lowering_matmul_back, hadamard_matmul.py:143-161):
    per sample, x_b <- P x_b then quantise with a step of its own.  Stochastic rounding numbers the
    elements as the flattened [B T, I] call does.  Returns (xq int8 [B, T', I], sx fp32 [B])."""
    x = np.asarray(x, dtype=F32)
    B, T, I = x.shape
    rows = np.asarray(cfg.hla_rows)
    nbs = T // cfg.hla_n
    idx_all = colwise_rng_index(I, B * nbs, rows)                       # [I, B nbs r]
    per = nbs * len(rows)
    xq, sx = [], []
    for b in range(B):
        xp = fwht_blocks_first(x[b], cfg.hla_n, rows)
        q, s = quant(xp, cfg.act_bits, cfg.act_scale, cfg.act_round, cfg.seed, STREAM_ACT,
                     index=idx_all[:, b * per:(b + 1) * per].T)
        xq.append(q)
        sx.append(s[0])
    return np.stack(xq), np.asarray(sx, dtype=F32)


def linear_backward_batched(g_y: np.ndarray, w: np.ndarray, xq: np.ndarray, sx: np.ndarray, cfg: HotConfig,
                            gw_ranges: int = 1):
    """FLinearQ.backward on 3-D tensors (quant_matmul.py:215-348): the g_y quantisers run per sample
    (per-tensor steps become per-sample steps; per-row steps stay per token for g_y H and become per
    sample and channel for (P g_y)^T), W has one step, grad_input is computed per sample and the
    per-sample weight gradients ((acc_b s_gw,b) s_x,b) are added up in fp32 (autograd's sum over
    the batch dimension of the returned [B, O, I] tensor, whose order torch leaves open), then
    divided by n.  The order here: the samples form gw_ranges ranges of ceil(B / gw_ranges)
    consecutive samples; each range is summed in sample order starting from zero, and the range
    sums are added in range order (gw_ranges = 1: plain sample order).
    Returns (g_x [B, T, I], g_w [O, I], list of per-sample traces)."""
    g_y = np.asarray(g_y, dtype=F32)
    w = np.asarray(w, dtype=F32)
    B, T, O = g_y.shape
    I = w.shape[1]
    rows = np.asarray(cfg.hla_rows)
    nbs = T // cfg.hla_n
    per = nbs * len(rows)
    Wh = fwht_blocks_first(w, cfg.n_o)
    qW, sW = quant(Wh, cfg.w_bits, cfg.w_scale, cfg.w_round, cfg.seed, STREAM_W,
                   index=colwise_rng_index(Wh.shape[1], Wh.shape[0] // cfg.n_o, np.arange(cfg.n_o)).T)
    gw_idx = colwise_rng_index(O, B * nbs, rows)                         # [O, B nbs r]
    g_x = np.empty((B, T, I), dtype=F32)
    per_range = -(-B // max(1, int(gw_ranges)))
    range_sums = []
    g_w = np.zeros((O, I), dtype=F32)
    traces = []
    for b in range(B):
        if b % per_range == 0 and b > 0:
            range_sums.append(g_w)
            g_w = np.zeros((O, I), dtype=F32)
        tr = BackwardTrace()
        G = fwht_blocks_last(g_y[b], cfg.n_o)
        gx_idx = (np.arange(b * T, (b + 1) * T, dtype=np.int64)[:, None] * O + np.arange(O, dtype=np.int64)[None, :])
        tr.qG, tr.sG = quant(G, cfg.gx_bits, cfg.gx_scale, cfg.gx_round, cfg.seed, STREAM_GX, index=gx_idx)
        tr.acc_x = int_gemm_nt(tr.qG, qW.T)
        sg = tr.sG.reshape(-1, 1) if cfg.gx_scale == SCALE_ROW else tr.sG.reshape(1, 1)
        g_x[b] = (((tr.acc_x.astype(F32) * sg).astype(F32) * sW[0]).astype(F32) / F32(cfg.n_o)).astype(F32)
        GpT = np.ascontiguousarray(fwht_blocks_first(g_y[b], cfg.hla_n, rows).T)           # [O, T']
        tr.qGp, tr.sGp = quant(GpT, cfg.gw_bits, cfg.gw_scale, cfg.gw_round, cfg.seed, STREAM_GW,
                               index=gw_idx[:, b * per:(b + 1) * per])
        tr.acc_w = int_gemm_nt(tr.qGp, np.asarray(xq[b]).T)
        sgw = tr.sGp.reshape(-1, 1) if cfg.gw_scale == SCALE_ROW else tr.sGp.reshape(1, 1)
        g_w = (g_w + ((tr.acc_w.astype(F32) * sgw).astype(F32) * F32(sx[b])).astype(F32)).astype(F32)
        traces.append(tr)
    range_sums.append(g_w)
    g_w = range_sums[0]
    for part in range_sums[1:]:
        g_w = (g_w + part).astype(F32)
    g_w = (g_w / F32(cfg.hla_n)).astype(F32)
    return g_x, g_w, traces
