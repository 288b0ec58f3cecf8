"""Op-for-op CPU port (PyTorch, float "fake quant") of the reference's HOT
linear layer, scheme gih_gwlr, as the reference itself evaluates it: dense
``torch.matmul`` transforms, float tensors holding integer values, global
torch RNG for stochastic rounding.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.  Used as
  * the CPU baseline timed by bench.py (``cpu_baseline.kind = "port"``), and
  * the second checker of the parity tests: the native fp32 g_x / g_W must be
    within 1e-3 relative Frobenius error of this port under round-to-nearest.
It differs from oracle/hot_oracle.py only in the summation order inside the
transform matmuls (BLAS instead of the canonical butterfly), i.e. in the last
ulp of the transformed values.

Restates /root/reference/utils/quant_matmul.py:19-31 (norm), :40-49 (sawb),
:86-100 (stoch), :108-116 (int), :178-212 (setup_context), :215-348
(backward) and utils/hadamard_matmul.py:121-161 (lowering matmuls).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import hot_oracle as orc

EPS = 1e-11


def _front(a: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
    """hadamard_matmul.py:121-141 (2-D)."""
    n = h.shape[0]
    return a @ h if a.shape[1] == n else (a.reshape(-1, n) @ h).reshape(a.shape[0], -1)


def _back(h: torch.Tensor, a: torch.Tensor) -> torch.Tensor:
    """hadamard_matmul.py:143-161 (2-D), including its two transposing copies."""
    if h.shape[1] == a.shape[0]:
        return h @ a
    return (a.T.reshape(-1, h.shape[1]) @ h.T).reshape(a.shape[1], -1).T


def _quant(x: torch.Tensor, bits: int, kind: str):
    qmax = 2 ** (bits - 1) - 1
    if kind == "int":                                    # :108-116
        mx = x.abs().max()
        s = mx / qmax
        return torch.round(torch.clamp(x, -mx, mx) / (s + EPS)), s
    if kind == "sawb":                                   # :40-49
        clip = 12.1 * torch.sqrt(torch.mean(x ** 2)) - 12.2 * torch.mean(x.abs())
        s = clip / qmax
        return torch.round(torch.clamp(x, -clip, clip) / (s + EPS)), s
    if kind in ("stoch", "nq"):                          # :86-100, :19-31
        mx = x.abs().max(dim=1, keepdim=True)[0] if kind == "nq" else x.abs().max()
        s = mx / qmax
        y = torch.clamp(x, -mx, mx) / (s + EPS)
        fl = torch.floor(y.abs())
        q = torch.sign(y) * (fl + torch.bernoulli(y.abs() - fl))
        return (q * s, 1.0) if kind == "nq" else (q, s)
    raise ValueError(kind)


@dataclass
class PortConfig:
    gx_bits: int = 4
    w_bits: int = 4
    gw_bits: int = 8
    act_bits: int = 8
    gx_kind: str = "int"
    w_kind: str = "int"
    gw_kind: str = "int"
    act_kind: str = "int"


def matrices(L: int, O: int, dtype=torch.float32):
    """hadamard_out (H_16 for O) and hadamard_bs (P for L), as HQ_Linear builds
    them (quant_matmul.py:365-367)."""
    h_out = torch.tensor(orc.make_hadamard(O), dtype=dtype)
    h_bs = torch.tensor(orc.make_WHT(L), dtype=dtype)
    return h_out, h_bs


def setup_context(x: torch.Tensor, h_bs: torch.Tensor, cfg: PortConfig):
    """quant_matmul.py:178-212: x <- P x, quantise, keep as int8."""
    xp = _back(h_bs, x)
    q, s = _quant(xp, cfg.act_bits, cfg.act_kind)
    return q.to(torch.int8), s


def backward(grad_output: torch.Tensor, w: torch.Tensor, xq: torch.Tensor, scale_x, h_out: torch.Tensor,
             h_bs: torch.Tensor, cfg: PortConfig, scheme: str = "gih_gwlr"):
    """quant_matmul.py:215-348, 2-D tensors, the branches of transform_scheme:
    "gih_gwlr" (h_out = block Hadamard of the out-features, h_bs = low-rank WHT rows of the tokens);
    "hadamard" (h_bs = the block Hadamard of make_hadamard for the token count: g_W branch :294-295, :338-339);
    "low_rank" (h_bs = low-rank WHT rows of the tokens for both products, W untransformed: :231-232, :263-264,
    :296-297, :334-335); "gilr_gwh" (h_out = low-rank WHT rows of the TOKENS for the g_x product, h_bs = block
    Hadamard of the tokens for the g_W product: :233-234, :265-266, :298-299, :336-338)."""
    if scheme in ("gih_gwlr", "hadamard"):
        g = _front(grad_output, h_out)                          # :230 / :238
        wh = _back(h_out, w)                                    # :262 / :270
    elif scheme == "low_rank":
        g = _back(h_bs, grad_output)                            # :232
        wh = w                                                  # :264
    elif scheme == "gilr_gwh":
        g = _back(h_out, grad_output)                           # :234
        wh = w                                                  # :266
    else:
        raise NotImplementedError(scheme)
    g, s_g = _quant(g, cfg.gx_bits, cfg.gx_kind)                # :244-257
    wh, s_w = _quant(wh, cfg.w_bits, cfg.w_kind)                # :276-285
    grad_input = (g @ wh) * s_g * s_w                           # :288-290
    if scheme in ("hadamard", "gilr_gwh"):
        gp = _front(grad_output.T.contiguous(), h_bs)           # :295 / :299
    else:
        gp = _back(h_bs, grad_output).T                         # :297 / :301
    gp, s_gp = _quant(gp, cfg.gw_bits, cfg.gw_kind)             # :307-320
    grad_w = (gp @ xq.to(gp.dtype)) * s_gp * scale_x            # :322-324
    if scheme == "hadamard":
        grad_input = grad_input / orc.pow2_factor_max16(h_out.shape[0])      # :331
        grad_w = grad_w / orc.pow2_factor_max16(h_bs.shape[0])               # :332
    elif scheme == "low_rank":
        grad_input = _back(h_bs.T.contiguous(), grad_input) / orc.pow2_factor(h_bs.shape[1])     # :334
        grad_w = grad_w / orc.pow2_factor(h_bs.shape[1])                     # :335
    elif scheme == "gilr_gwh":
        grad_input = _back(h_out.T.contiguous(), grad_input) / orc.pow2_factor(h_out.shape[1])   # :337
        grad_w = grad_w / orc.pow2_factor_max16(h_bs.shape[0])               # :338
    else:
        grad_input = grad_input / orc.pow2_factor_max16(h_out.shape[0])      # :343
        grad_w = grad_w / orc.pow2_factor(h_bs.shape[1])                     # :344
    return grad_input, grad_w


def config1_inputs(L: int = 12608, O: int = 3072, I: int = 768, seed: int = 0):
    """The CPU-runnable configuration: x ~ N(0,1) [L, I]; W = nn.Linear(I, O)
    weight (kaiming-uniform); g_y ~ N(0, 1e-3) [L, O]; torch.manual_seed(seed)."""
    torch.manual_seed(seed)
    x = torch.randn(L, I)
    w = torch.nn.Linear(I, O).weight.detach().clone()
    gy = 1e-3 * torch.randn(L, O)
    return x, w, gy
