"""Layer-wise quantizer selection (LQS): one calibration pass in full precision,
then, per layer, the choice between the per-tensor and the per-token stochastic
quantiser for the g_y operand of the g_x product.

Follows the reference's calibration worker (ViT_main.py:41-56 hooks,
:126-215 selection) and its two candidate quantisers
(utils/quant_matmul.py:19-37 norm_quantizer, :86-106 stoch_quantizer).  The
pass runs once before training on a handful of batches: it is host logic in
plain PyTorch, not part of the per-step path, and uses torch's generator for
the Bernoulli draws exactly as the reference does.

The result lands in ``args.layer_quant_dict`` under ``<layer>_gx`` and
``<layer>_gw``, where ``hot_amd.quant_matmul.options_for`` reads it when
``args.quantAuto`` is on.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, Optional

import torch
import torch.nn as nn

from . import args

quantScheme_gx = ("stoch_quantizer", "norm_quantizer")   # candidates, in the reference's order


def _stochastic_codes(y: torch.Tensor, generator=None) -> torch.Tensor:
    """sign(y) * (floor|y| + Bernoulli(frac|y|))."""
    mag = y.abs()
    low = torch.floor(mag)
    up = torch.rand(mag.shape, device=mag.device, dtype=mag.dtype, generator=generator) < (mag - low)
    return torch.sign(y) * (low + up.to(mag.dtype))


def stoch_quantizer(x: torch.Tensor, quantBits: int, is_batched: bool, generator=None):
    """One absmax step per tensor (per sample for 3-D input); returns (codes, step)."""
    qmax = 2 ** (quantBits - 1) - 1
    if is_batched:
        mx = x.abs().flatten(1).amax(dim=1)
        s = mx / qmax
        mxb, sb = mx.view(-1, 1, 1), s.view(-1, 1, 1)
    else:
        mx = x.abs().max()
        s = mx / qmax
        mxb, sb = mx, s
    y = torch.maximum(torch.minimum(x, mxb), -mxb) / (sb + args.eps)
    return _stochastic_codes(y, generator), s


def norm_quantizer(x: torch.Tensor, quantBits: int, is_batched: bool, generator=None):
    """One absmax step per row (dim 1 of each 2-D sample); returns (dequantised tensor, 1.0)."""
    qmax = 2 ** (quantBits - 1) - 1
    # rows of a 2-D sample are dim 0 entries with the max taken over dim 1; for [B, L, C] input each
    # sample is an [L, C] matrix, so the max runs over the last dim in both cases
    mx = x.abs().amax(dim=-1, keepdim=True)
    s = mx / qmax
    y = torch.maximum(torch.minimum(x, mx), -mx) / (s + 1e-11)
    return _stochastic_codes(y, generator) * s, 1.0


_CANDIDATES: Dict[str, Callable] = {"stoch_quantizer": stoch_quantizer, "norm_quantizer": norm_quantizer}


def quantisation_error(grad: torch.Tensor, scheme: str, bits: int = 4, generator=None) -> float:
    """Euclidean distance between a gradient and its quantise -> dequantise image."""
    batched = grad.dim() == 3
    q, s = _CANDIDATES[scheme](grad, bits, batched, generator)
    if batched and torch.is_tensor(s):
        s = s.view(-1, 1, 1)
    return float(torch.dist(grad, q * s))


def select_for_layer(grad: torch.Tensor, bits: int = 4, generator=None):
    """(gx scheme, gw scheme) for one layer's output gradient.

    The per-tensor quantiser is the default; the per-token one replaces it for g_x only when it
    more than halves the error, and g_W then keeps the per-tensor quantiser (ViT_main.py:194-211).
    """
    best = 9999.0
    gx = gw = None
    for scheme in quantScheme_gx:
        err = quantisation_error(grad, scheme, bits, generator)
        if err < best and scheme != "norm_quantizer":
            best, gx, gw = err, scheme, scheme
        elif err < best and (best - err) > best * 0.5:
            best, gx, gw = err, scheme, "stoch_quantizer"
    return gx, gw


class GradCapture:
    """Keeps, per hooked layer, the output gradient (and weight) of the FIRST backward pass that
    reaches it: the role of the reference's tensor dictionary during calibration (ViT_main.py:41-56),
    whose register() returns early once a slot is filled (utils/plot.py:175-177), so that the
    selection judges the gradients before any weight update.  ``keep="last"`` keeps the most recent
    pass instead."""

    def __init__(self, model: nn.Module, layer_types, keep: str = "first") -> None:
        if keep not in ("first", "last"):
            raise ValueError("keep must be 'first' or 'last'")
        self.keep = keep
        self.grads: Dict[str, torch.Tensor] = {}
        self.weights: Dict[str, torch.Tensor] = {}
        self._handles = []
        for name, module in model.named_modules():
            if isinstance(module, tuple(layer_types)):
                self._handles.append(module.register_full_backward_hook(self._hook(name, module)))

    def _hook(self, name, module):
        def fn(_mod, _grad_in, grad_out):
            if self.keep == "first" and name in self.grads:
                return
            self.grads[name] = grad_out[0].detach()
            self.weights[name] = module.weight.detach()
        return fn

    def close(self) -> None:
        for h in self._handles:
            h.remove()
        self._handles = []


def _as_tokens(grad: torch.Tensor) -> torch.Tensor:
    # convolution outputs [B, C, H, W] are judged as [B, H*W, C] token matrices (ViT_main.py:185-188)
    if grad.dim() > 3:
        B, C, H, W = grad.shape
        return grad.permute(0, 2, 3, 1).reshape(B, H * W, C)
    return grad


def calibrate(model: nn.Module, batches: Iterable, criterion: Callable, optimizer: Optional[torch.optim.Optimizer] = None,
              layer_types=None, bits: int = 4, generator=None, keep: str = "first") -> Dict[str, str]:
    """Runs the calibration batches through `model` with the HOT path switched off (full-precision
    backward), then fills and returns ``args.layer_quant_dict``.

    `batches` yields (inputs, target) pairs already on the model's device; the selection judges the
    gradients of the first batch, as the reference does (``keep="last"``: of the last one).  The
    quantiser and transform flags of ``args`` are restored afterwards."""
    from .quant_matmul import HQ_Conv2d, HQ_Linear
    layer_types = layer_types or (HQ_Linear, HQ_Conv2d)
    saved = {k: getattr(args, k) for k in ("TransformGogi", "TransformWgt", "TransformGogw", "TransformInput",
                                           "quantBWDGogi", "quantBWDWgt", "quantBWDGogw", "quantBWDAct", "quantAuto")}
    cap = GradCapture(model, layer_types, keep)
    try:
        args.TransformGogi = args.TransformWgt = args.TransformGogw = args.TransformInput = False
        args.quantBWDGogi = args.quantBWDWgt = args.quantBWDGogw = args.quantBWDAct = "no"
        args.quantAuto = False
        for inputs, target in batches:
            if optimizer is not None:
                optimizer.zero_grad()
            loss = criterion(model(inputs), target)
            loss.backward()
            if optimizer is not None:
                optimizer.step()
    finally:
        cap.close()
        for k, v in saved.items():
            setattr(args, k, v)
    for name, grad in cap.grads.items():
        gx, gw = select_for_layer(_as_tokens(grad).float(), bits, generator)
        if gx is not None:
            args.layer_quant_dict[name + "_gx"] = gx
            args.layer_quant_dict[name + "_gw"] = gw
    return args.layer_quant_dict
