"""Drop-in for the reference's compiled op module ``HLQ_backward``
(cuda_measure/HLQ_backward.cpp:6-24, backward_cuda in
cuda_measure/HLQ_backward_kernel.cu:457-737; call sites
cuda_measure/measure.py:65,72):

    gx, gw, time_list = HLQ_backward.backward(Go, W, X, 0, 0, 16, True)

Same arguments, checks, output shapes/dtypes and a 4-element list of seconds.
Unlike the reference op, whose GEMMs run on zero dummies with unit scales, the
results are the real HOT gradients (numerics of FLinearQ.backward, scheme
gih_gwlr).  The op transforms and quantises X itself, as the reference op does.
"""
from __future__ import annotations

from typing import List, Tuple

import torch

from . import ops
from .hadamard_matmul import hla_rows

# Quantiser choices of the op (the reference op hard-codes INT4 with stochastic
# rounding for the g_x operands and INT8 for the g_W operands).
gx_bits = 4
gw_bits = 8
gx_rounding = "stoch"
other_rounding = "nearest"
hla_max_block = 8192     # see hot_amd.args.hla_max_block
seed = 0


def _check(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor!" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous!" % name)
    if t.dim() != 2:
        raise RuntimeError("%s must be 2D!" % name)


def options(L: int, H_size: int, per_token: bool) -> ops.HotOptions:
    n, rows = hla_rows(L)
    if n > hla_max_block:
        n, rows = hla_rows(hla_max_block)
    return ops.HotOptions(
        n_o=int(H_size), hla_n=int(n), hla_rows=tuple(int(v) for v in rows),
        gx_bits=gx_bits, w_bits=gx_bits, gw_bits=gw_bits, act_bits=gw_bits,
        gx_round=gx_rounding, w_round=other_rounding, gw_round=other_rounding, act_round=other_rounding,
        gx_scale="row" if per_token else "tensor", seed=seed)


def backward(Go: torch.Tensor, W: torch.Tensor, X: torch.Tensor, reorder_idx_go=0, reorder_idx_X=0,
             H_size: int = 16, per_token: bool = True) -> Tuple[torch.Tensor, torch.Tensor, List[float]]:
    """Go [L, O], W [O, I], X [L, I] -> (gx [L, I], gw [O, I], [t0, t1, t2, t3]).

    ``reorder_idx_*`` are accepted and ignored, as in the reference (its C++
    never dereferences them).  time_list follows the reference's
    [fwht, quant, gemm, dequant] (HLQ_backward_kernel.cu:729-733) as far as
    fused kernels allow: seconds spent in {the transform passes that only
    measure (statistics of Go and W), the transform + quantise passes (Go
    twice, W, X), both GEMMs, 0.0 -- dequantisation is the GEMMs' epilogue},
    measured with HIP events on the current stream; their sum is the op's
    device time."""
    _check(Go, "Go")
    _check(W, "Wt")
    _check(X, "X")
    L, O = Go.shape
    if W.shape[0] != O or X.shape[0] != L or X.shape[1] != W.shape[1]:
        raise RuntimeError("shape mismatch: Go [L,O], W [O,I], X [L,I] expected")
    if H_size not in (16, 32, 64):
        raise RuntimeError("H_size must be 16, 32 or 64")
    opt = options(L, H_size, bool(per_token))
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    xq, sx = ops.abc_forward(X.to(Go.dtype) if X.dtype != Go.dtype else X, opt)
    e1.record()
    gx, gw, t = ops.linear_backward(Go, W, xq, sx, opt, timing=True)
    t[1] += e0.elapsed_time(e1) * 1e-3
    return gx, gw, t
