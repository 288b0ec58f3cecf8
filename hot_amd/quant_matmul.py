"""FLinearQ / HQ_Linear on the native gfx950 path.

Same class names, argument order and attributes as the reference's
utils/quant_matmul.py:169-422, so that
``replace_layers(model, nn.Linear, HQ_Linear)`` (utils/utils.py:53-74) works
unchanged.  Forward stays full precision (:173-175); ``setup_context`` writes
the INT8 Hadamard-compressed activation buffer (:178-212) with the native
kernel and ``backward`` (:215-348, scheme gih_gwlr) calls the fused native op.
``HQ_Conv2d`` (:426-488) lowers a convolution to the same Function by im2col.

With every Transform* flag off and every quantBWD* flag "no" the reference's
Function is an ordinary full-precision linear layer (its branches all fall
through); that setting is kept, because the layer-wise quantizer selection
calibrates in it.  Any other partial setting raises: there is no eager
stand-in for the HOT path, and on a CPU tensor the native path raises.
"""
from __future__ import annotations

from typing import Optional, Tuple

import threading
from dataclasses import replace

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor
from torch.autograd.function import Function

from . import args
from . import ops
from .hadamard_matmul import (Transform_Dict, biggest_power2_factor, biggest_power2_factor_max16, hla_rows,
                              paper_rows, run_major)

TD = Transform_Dict()

_QUANT_SCHEMES = {
    # name in args.layer_quant_dict -> (rounding, scale mode)
    "int_quantizer": (ops.ROUND_NEAREST, ops.SCALE_TENSOR),
    "stoch_quantizer": (ops.ROUND_STOCH, ops.SCALE_TENSOR),
    "norm_quantizer": (ops.ROUND_STOCH, ops.SCALE_ROW),
    "sawb_quantizer": (ops.ROUND_NEAREST, ops.SCALE_SAWB),
    # the logarithmic quantiser has entry points of its own (ops.gx_luq for the g_x product, see
    # gx_uses_luq; ops.gw_luq for the g_W product, see gw_uses_luq); the pair below only fills the option
    # fields those entry points do not read
    "luq_quantizer": (ops.ROUND_STOCH, ops.SCALE_TENSOR),
}
_FLAG_SCHEMES = {"int": "int_quantizer", "stoch": "stoch_quantizer", "nq": "norm_quantizer",
                 "sawb": "sawb_quantizer", "luq": "luq_quantizer"}


def gx_uses_luq(layer_name: str = " ") -> bool:
    """True when the g_y quantiser of the g_x product is luq_quantizer (args.quantBWDGogi == "luq", or the
    layer's entry of args.layer_quant_dict under quantAuto; utils/quant_matmul.py:244-253)."""
    if args.quantAuto and len(args.layer_quant_dict) > 0:
        return args.layer_quant_dict.get(layer_name + "_gx") == "luq_quantizer"
    return args.quantBWDGogi == "luq"


def gw_uses_luq(layer_name: str = " ") -> bool:
    """True when the quantiser of the projected g_y of the g_W product is luq_quantizer
    (args.quantBWDGogw == "luq", or the layer's "_gw" entry under quantAuto; utils/quant_matmul.py:307-314)."""
    if args.quantAuto and len(args.layer_quant_dict) > 0:
        return args.layer_quant_dict.get(layer_name + "_gw") == "luq_quantizer"
    return args.quantBWDGogw == "luq"


def _scheme(flag: str, what: str, allowed) -> Tuple[int, int]:
    if flag not in allowed:
        raise NotImplementedError("%s rounding scheme %r is not implemented on the native path (use one of %s)"
                                  % (what, flag, sorted(allowed)))
    return _QUANT_SCHEMES[_FLAG_SCHEMES[flag]]


def token_rule(tokens: int):
    """(n, rows) of the token-wise transform for a token count: the low-rank projection under
    args.hla_rule, or, with the reference's scheme "hadamard", the whole block Hadamard of make_hadamard
    along the tokens (utils/quant_matmul.py:182-183,294-295,353-355: every coefficient, natural order)."""
    if args.transform_scheme in ("hadamard", "gilr_gwh"):
        # "gilr_gwh": the g_W product and the activation buffer use the whole block Hadamard
        # (utils/quant_matmul.py:186-187,298-299); its g_x product the projection of gx_token_rule
        n = int(biggest_power2_factor_max16(int(tokens)))
        return n, np.arange(n)
    if args.hla_rule == "paper":
        if tokens % 16:
            return 1, np.array([0])
        return paper_rows(16, 8)
    n, rows = hla_rows(tokens, args.vectorPercentile)
    if n > args.hla_max_block:
        n, rows = hla_rows(args.hla_max_block, args.vectorPercentile)
    if n > 128:
        # the two-level kernels store the codes themselves when the rows come run by run; the order along
        # K is shared by the activation buffer and the gradient operand and cancels in their product
        rows = run_major(rows)
    return n, rows


LOWRANK_GX_SCHEMES = ("low_rank", "gilr_gwh")


def gx_token_rule(tokens: int):
    """(n, rows) of the projection P along the tokens that the schemes "low_rank" and "gilr_gwh" apply to
    g_y for the g_x product (utils/quant_matmul.py:229-233; P is make_WHT of the token count, :356-362):
    the low-rank rule of args.hla_rule, blocks of up to args.hla_max_block tokens as for the g_W side."""
    if args.hla_rule == "paper":
        return (1, np.array([0])) if tokens % 16 else paper_rows(16, 8)
    n, rows = hla_rows(tokens, args.vectorPercentile)
    if n > args.hla_max_block:
        n, rows = hla_rows(args.hla_max_block, args.vectorPercentile)
    return n, rows


def hot_switched_off() -> bool:
    """True when args describes the reference's plain full-precision layer: no transform, no
    quantiser (the state of args.py:40-49 before a recipe is applied)."""
    off = (False, "no", None)
    return (not (args.TransformGogi or args.TransformWgt or args.TransformGogw or args.TransformInput)
            and all(getattr(args, k) in off for k in ("quantBWDGogi", "quantBWDWgt", "quantBWDGogw", "quantBWDAct")))


_OPTIONS_CACHE: dict = {}


def options_for(tokens: int, layer_name: str = " ", out_features: int = 16) -> ops.HotOptions:
    """args.* -> HotOptions, following the branch structure of FLinearQ.  The Hadamard block along the
    out-features is the reference's make_hadamard rule: the largest power of two dividing them, at
    most 16 (utils/hadamard_matmul.py:57-59): 16 for the usual widths, 4 for a 100-class head.
    The result is cached per state of the flags it reads (layers call this on every step)."""
    auto = bool(args.quantAuto and len(args.layer_quant_dict) > 0)
    key = (tokens, out_features, args.transform_scheme, args.TransformGogi, args.TransformWgt, args.TransformGogw,
           args.TransformInput, args.quantBWDGogi, args.quantBWDWgt, args.quantBWDGogw, args.quantBWDAct,
           args.GogiQuantBit, args.weightQuantBit, args.GogwQuantBit, args.actQuantBit, args.hla_rule,
           args.hla_max_block, args.vectorPercentile,
           (args.layer_quant_dict.get(layer_name + "_gx"), args.layer_quant_dict.get(layer_name + "_gw")) if auto else None)
    seed = (int(args.sr_seed) << 20) + int(args.sr_step)
    hit = _OPTIONS_CACHE.get(key)
    if hit is not None:
        return hit.with_seed(seed)
    if len(_OPTIONS_CACHE) > 4096:
        _OPTIONS_CACHE.clear()
    opt = _options_uncached(tokens, layer_name, out_features)
    _OPTIONS_CACHE[key] = opt
    return opt.with_seed(seed)


def _options_uncached(tokens: int, layer_name: str, out_features: int) -> ops.HotOptions:
    # "hadamard" differs from "gih_gwlr" in the token-wise transform only (token_rule); "low_rank" and
    # "gilr_gwh" project g_y along the tokens for the g_x product as well (gx_token_rule, ops.gx_lowrank);
    # "gilro_gwh" projects along the out-features and has no activation branch in the reference's
    # setup_context (utils/quant_matmul.py:181-192 raises for it): not built
    if args.transform_scheme not in ("gih_gwlr", "hadamard") + LOWRANK_GX_SCHEMES:
        raise NotImplementedError("transform scheme %r: gih_gwlr, hadamard, low_rank and gilr_gwh run natively"
                                  % args.transform_scheme)
    if not (args.TransformGogi and args.TransformWgt and args.TransformGogw and args.TransformInput):
        raise NotImplementedError("the native path needs all four Transform* flags on")
    n, rows = token_rule(tokens)
    gx_bits, gw_bits = args.GogiQuantBit, args.GogwQuantBit
    if args.quantAuto and len(args.layer_quant_dict) > 0:
        # utils/quant_matmul.py:244-245 and :307-308 (the g_W branch reads GogiQuantBit there)
        gx_round, gx_scale = _QUANT_SCHEMES[args.layer_quant_dict[layer_name + "_gx"]]
        gw_round, gw_scale = _QUANT_SCHEMES[args.layer_quant_dict[layer_name + "_gw"]]
        gw_bits = args.GogiQuantBit
    else:
        gx_round, gx_scale = _scheme(args.quantBWDGogi, "GradHo", ("int", "stoch", "nq", "luq"))
        gw_round, gw_scale = _scheme(args.quantBWDGogw, "GradHb", ("int", "stoch", "nq", "luq"))
    w_round, w_scale = _scheme(args.quantBWDWgt, "Weight", ("int", "stoch", "sawb"))
    act_round, act_scale = _scheme(args.quantBWDAct, "Activation", ("int", "stoch", "sawb"))
    return ops.HotOptions(
        n_o=int(biggest_power2_factor_max16(int(out_features))), hla_n=int(n), hla_rows=tuple(int(v) for v in rows),
        gx_bits=gx_bits, w_bits=args.weightQuantBit, gw_bits=gw_bits, act_bits=args.actQuantBit,
        gx_round=gx_round, w_round=w_round, gw_round=gw_round, act_round=act_round,
        gx_scale=gx_scale, w_scale=w_scale, gw_scale=gw_scale, act_scale=act_scale,
        seed=(int(args.sr_seed) << 20) + int(args.sr_step))


def _check_padding(w: Tensor, opt: ops.HotOptions) -> None:
    if (w.shape[0] % 8 or w.shape[1] % 8) and ops.SCALE_SAWB in (opt.w_scale, opt.act_scale):
        raise NotImplementedError("SAWB statistics over zero-padded channels would differ from the reference: "
                                  "feature counts must be multiples of 8 with the sawb quantisers")


def _pad8(t: Tensor) -> Tensor:
    """`t` contiguous, its last dimension padded with zeros to a multiple of 8."""
    extra = (-t.shape[-1]) % 8
    return F.pad(t, (0, extra)).contiguous() if extra else t.contiguous()


# torch keeps the transform check where Function.apply itself reads it; without it the class falls
# back to the stock apply
_PLAIN_APPLY = hasattr(torch._C, "_are_functorch_transforms_active")


# The activation buffer is written beside the forward GEMM, not behind it: the two read the same x and
# neither needs the other (the GEMM is bound by the matrix cores, the buffer kernels by memory).
# forward() records an event on the current stream before it launches the GEMM; setup_context, which
# autograd calls right after forward on the same thread, lets a side stream wait for that event, runs
# the buffer kernels there and makes the current stream wait for them.  One side stream per device,
# default priority.  Not under stream capture (a capture must not be forked behind its back).
_FWD = threading.local()
_SIDE_STREAMS: dict = {}
overlap_buffer_write = True


def _mark_input_ready(x: Tensor) -> None:
    _FWD.event = None
    if not (overlap_buffer_write and x.is_cuda) or hot_switched_off() or torch.cuda.is_current_stream_capturing():
        return
    ev = torch.cuda.Event()
    ev.record()
    _FWD.event = (ev, x.data_ptr())


def _buffer_stream(x: Tensor):
    """The side stream for the buffer kernels of this layer, already waiting for x; None = run in line."""
    mark = getattr(_FWD, "event", None)
    _FWD.event = None
    if mark is None or mark[1] != x.data_ptr():
        return None
    key = x.device.index
    side = _SIDE_STREAMS.get(key)
    if side is None:
        side = _SIDE_STREAMS[key] = torch.cuda.Stream(device=x.device)
    side.wait_event(mark[0])
    return side


class FLinearQ(Function):
    """torch.autograd.Function with the reference's forward / setup_context /
    backward triple (utils/quant_matmul.py:169-348)."""

    @classmethod
    def apply(cls, x, w, h_out, h_bs, name, bias=None):
        # Function.apply inspects the signature of forward on every call to fill in defaults
        # (about 30 us); with all six arguments in hand there is nothing to fill in
        if _PLAIN_APPLY and not torch._C._are_functorch_transforms_active():
            return super(Function, cls).apply(x, w, h_out, h_bs, name, bias)
        return super().apply(x, w, h_out, h_bs, name, bias)

    @staticmethod
    def forward(x, w, h_out, h_bs, name, bias=None):
        # `bias` is an addition to the reference's five arguments (which adds the bias after the
        # Function, utils/quant_matmul.py:419-420): inside, it rides in the GEMM epilogue instead of
        # costing a pass over the output
        _mark_input_ready(x)
        return F.linear(x, w, bias)

    @staticmethod
    def setup_context(ctx, inputs, output):
        x, w, _h_out, _h_bs, name = inputs[:5]
        ctx.has_bias = len(inputs) > 5 and inputs[5] is not None
        ctx.name = name
        ctx.x_shape = tuple(x.shape)
        ctx.full_precision = hot_switched_off()
        if ctx.full_precision:
            ctx.save_for_backward(x, w)
            return
        # the kernels move 16-byte vectors: feature counts that are not multiples of 8 are padded with
        # zero channels, which change neither a Hadamard block of the real channels nor any absmax
        ctx.batched = False
        side = _buffer_stream(x)
        if x.dim() == 3 and args.batched_mode == "per_sample":
            # the reference's treatment of 3-D activations: every sample has steps of its own
            tokens = x.shape[1]
            opt = options_for(tokens, name, w.shape[0])
            _check_padding(w, opt)
            if opt.hla_n <= 128:
                # one call per layer: the library keeps the samples apart
                ctx.batched = True
                xq, sx = ops.abc_forward_batched(_pad8(x), opt, side=side if x.shape[-1] % 8 == 0 and x.is_contiguous() else None)
            else:
                bufs = [ops.abc_forward(_pad8(x[b]), opt) for b in range(x.shape[0])]
                xq = torch.stack([b[0] for b in bufs])
                sx = torch.cat([b[1] for b in bufs])
        else:
            x2 = x.reshape(-1, x.shape[-1])
            opt = options_for(x2.shape[0], name, w.shape[0])
            _check_padding(w, opt)
            xq, sx = ops.abc_forward(_pad8(x2), opt, side=side if x2.shape[-1] % 8 == 0 and x2.data_ptr() == x.data_ptr() and x2.is_contiguous() else None)
        ctx.opt = opt
        args.sr_step += 1
        ctx.save_for_backward(xq, w, sx)

    @staticmethod
    def backward(ctx, grad_output):
        if ctx.full_precision:
            x, w = ctx.saved_tensors
            go = grad_output.to(w.dtype)
            grad_w = go.mT @ x.to(w.dtype)
            if grad_w.dim() == 3:                    # [B, O, I]: the sum over samples autograd would take
                grad_w = grad_w.sum(dim=0)
            return go @ w, grad_w, None, None, None, FLinearQ._bias_grad(ctx, grad_output)
        xq, w, sx = ctx.saved_tensors
        opt = ctx.opt
        go = grad_output
        O, I = w.shape
        wc = _pad8(_pad8(w).t()).t().contiguous() if (O % 8 or I % 8) else w.contiguous()   # [O8, I8]
        if go.dtype != wc.dtype:
            go = go.to(wc.dtype)
        luq = gx_uses_luq(ctx.name)
        luq_gw = gw_uses_luq(ctx.name)
        if args.transform_scheme in LOWRANK_GX_SCHEMES or luq or luq_gw:
            # g_x by an entry point of its own -- the projection along the tokens and its expansion
            # ("low_rank", "gilr_gwh"), or the logarithmic quantiser on g_y --, g_W as in "gih_gwlr" /
            # "hadamard": the token-wise kernel on g_y, then the INT8 product; or, with the logarithmic
            # quantiser on the projected g_y, ops.gw_luq
            # 3-D activations with a step per sample (the reference's vmap over the batch,
            # utils/quant_matmul.py:79-83): one pass per sample, sample b seeded with seed + b, the weight
            # gradients of the samples added in fp32 in sample order
            if luq and args.transform_scheme in LOWRANK_GX_SCHEMES:
                raise NotImplementedError("quantBWDGogi luq runs with the schemes gih_gwlr and hadamard")
            per_sample = go.dim() == 3 and args.batched_mode == "per_sample"
            samples = [go[b] for b in range(go.shape[0])] if per_sample else [go.reshape(-1, go.shape[-1])]
            gxs, gw = [], None
            for b, g in enumerate(samples):
                opt_b = replace(opt, seed=opt.seed + b) if b else opt
                go2 = _pad8(g)
                lp = (go2.shape[0] // opt.hla_n) * opt.hla_r
                if not per_sample:
                    xq_b, sx_b = xq, sx
                elif ctx.batched:
                    # the batched buffer keeps the samples side by side along K; the product reads whole
                    # 128-code stages, so the sample's codes move to a zero-padded operand of their own
                    kg = ops.kpad_group(go2.shape[0], opt)
                    xq_b = torch.zeros((xq.shape[0], ops.kpad(lp)), dtype=xq.dtype, device=xq.device)
                    xq_b[:, :lp] = xq[:, b * kg:b * kg + lp]
                    sx_b = sx[b:b + 1]
                else:
                    xq_b, sx_b = xq[b], sx[b:b + 1]
                if luq:
                    gx = ops.gx_luq(go2, wc, opt_b)
                elif args.transform_scheme in LOWRANK_GX_SCHEMES:
                    n_gx, rows_gx = gx_token_rule(go2.shape[0])
                    gx = ops.gx_lowrank(go2, wc, replace(opt_b, hla_n=int(n_gx), hla_rows=tuple(int(v) for v in rows_gx)))
                else:
                    # the usual g_x, from the fused call (its g_W, by the quantiser the option fields
                    # name for the logarithmic one, is dropped)
                    gx = ops.linear_backward(go2, wc, xq_b, sx_b, opt_b)[0]
                gw_dtype = torch.float32 if per_sample else wc.dtype
                if luq_gw:
                    gw_b = ops.gw_luq(go2, xq_b, sx_b, opt_b, out_dtype=gw_dtype)
                else:
                    qgp, sgp, lp = ops.hla_tokenwise(go2, opt.hla_n, opt.hla_rows, bits=opt.gw_bits,
                                                     rounding="stoch" if opt.gw_round == ops.ROUND_STOCH else "nearest",
                                                     scale="row" if opt.gw_scale == ops.SCALE_ROW else "tensor",
                                                     seed=opt_b.seed, rng_stream=ops.STREAM_GW)
                    # both operands hold one code per byte whatever their widths (the token-wise kernel and
                    # the activation buffer never pack): an INT8 product, as in the fused path
                    gw_b = ops.gemm_i8(qgp, xq_b, lp, 8, sgp, sx_b, post_scale=1.0 / opt.hla_n, out_dtype=gw_dtype)
                gw = gw_b if gw is None else gw + gw_b
                gxs.append(gx[:, :I])
            grad_w = gw.to(wc.dtype)
            grad_input = torch.stack(gxs) if per_sample else gxs[0].reshape(ctx.x_shape)
        elif go.dim() == 3 and args.batched_mode == "per_sample" and ctx.batched:
            gx, grad_w = ops.linear_backward_batched(_pad8(go), wc, xq, sx, opt)
            grad_input = gx[..., :I]
        elif go.dim() == 3 and args.batched_mode == "per_sample":
            gxs, gw = [], None
            for b in range(go.shape[0]):
                gx_b, gw_b = ops.linear_backward(_pad8(go[b]), wc, xq[b], sx[b:b + 1], opt)
                gxs.append(gx_b[:, :I])
                gw = gw_b.float() if gw is None else gw + gw_b.float()
            grad_input = torch.stack(gxs)
            grad_w = gw.to(wc.dtype)
        else:
            go2 = go.reshape(-1, go.shape[-1])
            if ctx.has_bias and ctx.needs_input_grad[5]:
                # the statistics pass over g_y holds the sum of every token block: the bias gradient
                # comes out of the same call instead of a reduction of its own over g_y
                gx, grad_w, gb = ops.linear_backward(_pad8(go2), wc, xq, sx, opt, bias_grad=True)
                grad_input = gx[:, :I].reshape(ctx.x_shape)
                if O % 8 or I % 8:
                    grad_w = grad_w[:O, :I]
                return grad_input, grad_w, None, None, None, gb[:O].to(grad_output.dtype)
            gx, grad_w = ops.linear_backward(_pad8(go2), wc, xq, sx, opt)
            grad_input = gx[:, :I].reshape(ctx.x_shape)
        if O % 8 or I % 8:
            grad_w = grad_w[:O, :I]
        return grad_input, grad_w, None, None, None, FLinearQ._bias_grad(ctx, grad_output)

    @staticmethod
    def _bias_grad(ctx, grad_output):
        if not (ctx.has_bias and ctx.needs_input_grad[5]):
            return None
        return grad_output.reshape(-1, grad_output.shape[-1]).sum(dim=0)


class HQ_Linear(nn.Linear):
    """nn.Linear whose backward runs the HOT path (utils/quant_matmul.py:350-422).

    ``hadamard_out`` (H_16 for the out-features) and ``hadamard_bs`` (the
    low-rank rows P for the token count) are kept as attributes for
    compatibility; they are non-persistent buffers because P depends on the
    token count of the batch at hand (the reference deletes them from
    checkpoints for that reason, ViT_main.py:302-304)."""

    def __init__(self, in_features, out_features, bias=True) -> None:
        super().__init__(in_features, out_features, bias)
        self.register_buffer("hadamard_out", torch.tensor(TD.get_or_register("hadamard", self.out_features),
                                                          dtype=self.weight.dtype), persistent=False)
        self.register_buffer("hadamard_bs", torch.ones((1, 1), dtype=self.weight.dtype), persistent=False)
        self._bs_tokens = None
        self.layer_name = " "

    def _refresh_bs(self, tokens: int) -> None:
        key = (tokens, args.transform_scheme, args.hla_rule, args.hla_max_block, args.vectorPercentile)
        if self._bs_tokens == key:
            return
        n, rows = token_rule(tokens)
        self._bs_tokens = key
        if n > 64:
            # the kernels take the row list, not the matrix: a block of 8192 tokens would make P
            # 2080 x 8192 per layer, so beyond 64 tokens the attribute is only a placeholder
            self.hadamard_bs = torch.ones((1, 1), dtype=self.weight.dtype, device=self.weight.device)
            return
        # P = rows of H_n
        idx = torch.tensor(np.array(rows), dtype=torch.long)
        i = idx[:, None] & torch.arange(n)[None, :]
        par = torch.zeros_like(i)
        while bool(i.any()):
            par ^= i & 1
            i >>= 1
        self.hadamard_bs = (1 - 2 * par).to(self.weight.dtype).to(self.weight.device)

    def forward(self, input: Tensor) -> Tensor:
        if input.dim() == 3 and args.batched_mode == "per_sample":
            self._refresh_bs(input.shape[1])
        else:
            self._refresh_bs(input.numel() // input.shape[-1])
        return FLinearQ.apply(input, self.weight, self.hadamard_out, self.hadamard_bs, self.layer_name, self.bias)


class HQ_Conv2d(nn.Conv2d):
    """nn.Conv2d (groups = 1) whose backward runs the HOT path: unfold to [B, H'W', C k k], the
    same Function as HQ_Linear with the weight viewed as [O, C k k], fold back
    (utils/quant_matmul.py:426-488).  Tokens are the output positions of one sample."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode="zeros") -> None:
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias, padding_mode)
        self.register_buffer("hadamard_out", torch.tensor(TD.get_or_register("hadamard", self.out_channels),
                                                          dtype=self.weight.dtype), persistent=False)
        self.register_buffer("hadamard_bs", torch.zeros((1, 1), dtype=self.weight.dtype), persistent=False)
        self.layer_name = " "

    def forward(self, input: Tensor) -> Tensor:
        if self.groups > 1:                          # depth-wise convolution
            raise NotImplementedError
        B, Cin, H, W = input.shape
        kh, kw = self.kernel_size
        if (tuple(self.stride) == (kh, kw) and tuple(self.padding) == (0, 0) and tuple(self.dilation) == (1, 1)
                and self.padding_mode == "zeros" and H % kh == 0 and W % kw == 0):
            # non-overlapping patches (a ViT patch embedding): unfold is a permutation, one copy
            # instead of the im2col kernel
            cols = (input.reshape(B, Cin, H // kh, kh, W // kw, kw).permute(0, 2, 4, 1, 3, 5)
                    .reshape(B, (H // kh) * (W // kw), Cin * kh * kw))
        else:
            cols = F.unfold(input, self.kernel_size, dilation=self.dilation, padding=self.padding,
                            stride=self.stride).transpose(1, 2)          # [B, H'W', C k k]
        weight = self.weight.view(self.weight.size(0), -1)
        output = FLinearQ.apply(cols, weight, self.hadamard_out, self.hadamard_bs, self.layer_name, self.bias)
        ho = (H + 2 * self.padding[0] - self.dilation[0] * (self.kernel_size[0] - 1) - 1) // self.stride[0] + 1
        wo = (W + 2 * self.padding[1] - self.dilation[1] * (self.kernel_size[1] - 1) - 1) // self.stride[1] + 1
        return output.transpose(1, 2).reshape(B, self.out_channels, ho, wo)
