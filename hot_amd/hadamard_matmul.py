"""Transform helpers with the names of the reference's utils/hadamard_matmul.py.

Host-side logic only (sizes, matrices, row selections); the hot path itself
never multiplies by these matrices -- the kernels run butterflies -- but the
matrices are what `HQ_Linear` exposes as `hadamard_out` / `hadamard_bs` and
what callers of the reference's helper API expect to get back.

Reference: utils/hadamard_matmul.py:9-59 (sizes, Sylvester matrix),
:121-161 (block-wise application), :167-178,209-226 (sequency-ordered
low-rank rows), :228-254 (cache).
"""
from __future__ import annotations

import functools
import math
from typing import Dict, Tuple

import numpy as np
import torch

__all__ = [
    "biggest_power2_factor", "biggest_power2_factor_max16", "hadamard", "make_hadamard",
    "make_WHT", "hla_rows", "paper_rows", "lowering_matmul_front", "lowering_matmul_back",
    "Transform_Dict",
]


def biggest_power2_factor(size_m: int) -> int:
    """Largest power of two dividing size_m (utils/hadamard_matmul.py:9-15)."""
    size_m = int(size_m)
    if size_m < 1:
        raise ValueError("size must be positive")
    return size_m & (-size_m)


def biggest_power2_factor_max16(size_m: int) -> int:
    """As above, limited to 16 for sizes above 16 (utils/hadamard_matmul.py:17-27)."""
    p = biggest_power2_factor(size_m)
    return 16 if (p > 16 and size_m > 16) else p


def hadamard(n: int) -> np.ndarray:
    """Sylvester Hadamard matrix of order n, natural order
    (utils/hadamard_matmul.py:32-51)."""
    n = int(n)
    if n < 1 or n & (n - 1):
        raise ValueError("n must be int and power of 2.")
    h = np.ones((1, 1), dtype=int)
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h


def make_hadamard(size_m: int) -> np.ndarray:
    """utils/hadamard_matmul.py:57-59."""
    return hadamard(biggest_power2_factor_max16(size_m))


def _sequency(n: int) -> np.ndarray:
    """Sign changes of each natural-order row: gray_decode(bit_reverse(i))."""
    bits = n.bit_length() - 1
    idx = np.arange(n, dtype=np.int64)
    rev = np.zeros(n, dtype=np.int64)
    for b in range(bits):
        rev |= ((idx >> b) & 1) << (bits - 1 - b)
    seq = rev.copy()
    shift = rev >> 1
    while shift.any():
        seq ^= shift
        shift >>= 1
    return seq


def _kept_sequencies(n: int, percentile: float) -> np.ndarray:
    """The zig-zag subset of utils/hadamard_matmul.py:215-225."""
    side = 1
    while (2 * side) ** 2 <= n:
        side *= 2
    sf = int(0.1 * (-np.sqrt(2 * side ** 2 * percentile + 25) + 10 * side + 5))
    every = np.arange(n)
    keep = []
    for band in range(side):
        lo, hi = side * band, side * (band + 1)
        keep.append(every[lo: hi - (band + sf)] if band % 2 == 0 else every[lo + (band + sf): hi])
    return np.concatenate(keep)


@functools.lru_cache(maxsize=256)
def _hla_rows_cached(n: int, percentile: float) -> np.ndarray:
    order = np.argsort(_sequency(n), kind="stable")   # natural row of each sequency
    rows = order[_kept_sequencies(n, percentile)]
    rows.setflags(write=False)                        # shared between callers
    return rows


def hla_rows(size_m: int, percentile: float = 50) -> Tuple[int, np.ndarray]:
    """(n, natural-order row of each kept coefficient) for a token count: the
    rule behind make_WHT, in the index form the kernels take (the array is cached and read-only)."""
    n = 1 if size_m == 1 else biggest_power2_factor(size_m)
    return n, _hla_rows_cached(int(n), float(percentile))


def run_major(rows) -> np.ndarray:
    """The same kept rows listed by (row % 64, row // 64).  The order of the kept coefficients is the
    order of the codes along K of both operands of the g_W product and does not show in its result; in
    this order the coefficients that one coefficient index of the 64-point stage of the two-level
    token-wise path yields are neighbours, and its quantise pass stores them K-major itself."""
    rows = np.asarray(rows)
    return rows[np.lexsort((rows // 64, rows % 64))]


def paper_rows(n: int = 16, r: int = 8) -> Tuple[int, np.ndarray]:
    """The r lowest sequencies of an n-block (utils/analysis_calculator.py:174-175)."""
    return n, np.argsort(_sequency(n), kind="stable")[:r]


def make_WHT(size_m: int, percentile: float = 50) -> np.ndarray:
    """Low-rank Walsh-Hadamard rows P (r x n) (utils/hadamard_matmul.py:209-226)."""
    n, rows = hla_rows(size_m, percentile)
    # rows of the Sylvester matrix in closed form, H[i, j] = (-1)^popcount(i & j),
    # so that a large n never materialises the full n x n matrix
    both = rows[:, None].astype(np.int64) & np.arange(n, dtype=np.int64)[None, :]
    parity = np.zeros_like(both)
    while both.any():
        parity ^= both & 1
        both >>= 1
    return (1 - 2 * parity).astype(int)


def lowering_matmul_front(A: torch.Tensor, H: torch.Tensor) -> torch.Tensor:
    """A times blockdiag(H) on the last dim (utils/hadamard_matmul.py:121-141)."""
    n = H.shape[0]
    if A.dim() not in (2, 3):
        raise NotImplementedError
    if A.shape[-1] == n:
        return A @ H
    lead = A.shape[:-1]
    return (A.reshape(*lead[:-1], -1, n) @ H).reshape(*lead, -1)


def lowering_matmul_back(H: torch.Tensor, A: torch.Tensor) -> torch.Tensor:
    """blockdiag(H) times A on dim -2 (utils/hadamard_matmul.py:143-161); H may
    be rectangular (r x n), output row index = block * r + k."""
    r, n = H.shape
    if A.dim() not in (2, 3):
        return A
    if A.shape[-2] == n:
        return H @ A
    cols = A.shape[-1]
    blocks = A.reshape(*A.shape[:-2], -1, n, cols)            # [.., nb, n, cols]
    return (H @ blocks).reshape(*A.shape[:-2], -1, cols)       # [.., nb*r, cols]


class Transform_Dict:
    """Process-wide cache name+size -> matrix (utils/hadamard_matmul.py:228-254)."""

    def __init__(self) -> None:
        self.transform_dict: Dict[str, np.ndarray] = {}

    def get(self, name: str, size: int) -> np.ndarray:
        return self.transform_dict[name + str(size)]

    def register(self, name: str, size: int, vectorPercentile: float = 50) -> None:
        if name == "hadamard":
            self.transform_dict[name + str(size)] = make_hadamard(size)
        elif name == "low_rank":
            self.transform_dict[name + str(size)] = make_WHT(size, vectorPercentile)
        else:
            raise NotImplementedError(name)

    def get_or_register(self, name: str, size: int, vectorPercentile: float = 50) -> np.ndarray:
        key = name + str(size)
        if key not in self.transform_dict:
            self.register(name, size, vectorPercentile)
        return self.transform_dict[key]
