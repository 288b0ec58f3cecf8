"""Torch-facing wrappers of the C ABI: tensors in, tensors out.

PyTorch is used for device memory (its caching allocator provides outputs and
workspaces, so nothing is hipMalloc'ed per call) and for the current stream;
all arithmetic happens in libhot_gfx950.so.
"""
from __future__ import annotations

import ctypes as C
import functools
from dataclasses import dataclass, field, replace
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import (BF16, F16, F32, ROUND_NEAREST, ROUND_STOCH, SCALE_ROW, SCALE_SAWB, SCALE_TENSOR,
                   STREAM_ACT, STREAM_GW, STREAM_GX, STREAM_W, HotError)

_DTYPES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_ROUND = {"nearest": ROUND_NEAREST, "int": ROUND_NEAREST, "stoch": ROUND_STOCH, "stochastic": ROUND_STOCH,
          ROUND_NEAREST: ROUND_NEAREST, ROUND_STOCH: ROUND_STOCH}
_SCALE = {"tensor": SCALE_TENSOR, "row": SCALE_ROW, "token": SCALE_ROW, "sawb": SCALE_SAWB,
          SCALE_TENSOR: SCALE_TENSOR, SCALE_ROW: SCALE_ROW, SCALE_SAWB: SCALE_SAWB}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError("unsupported dtype %s (float32, bfloat16 or float16)" % t.dtype)


def _need_gpu_2d(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor!" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous!" % name)
    if t.dim() != 2:
        raise RuntimeError("%s must be 2D!" % name)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ws(nbytes: int, device) -> torch.Tensor:
    # torch allocations are at least 512-byte aligned
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


@functools.lru_cache(maxsize=4096)
def kpad(k: int) -> int:
    return int(_lib.lib().hot_kpad(int(k)))


@dataclass(frozen=True)
class HotOptions:
    """Options of the fused path (struct hot_config); the fields FLinearQ reads
    from the reference's module-global ``args`` for scheme gih_gwlr."""
    n_o: int = 16
    hla_n: int = 1
    hla_rows: Sequence[int] = (0,)
    gx_bits: int = 4
    w_bits: int = 4
    gw_bits: int = 8
    act_bits: int = 8
    gx_round: int = ROUND_NEAREST
    w_round: int = ROUND_NEAREST
    gw_round: int = ROUND_NEAREST
    act_round: int = ROUND_NEAREST
    gx_scale: int = SCALE_TENSOR
    w_scale: int = SCALE_TENSOR
    gw_scale: int = SCALE_TENSOR
    act_scale: int = SCALE_TENSOR
    seed: int = 0
    streams: int = 0      # launch order of the backward: 0 = the library's rule, 1 = one stream, 2 = with its side stream

    @property
    def hla_r(self) -> int:
        return len(self.hla_rows)

    def lprime(self, L: int) -> int:
        return (L // self.hla_n) * self.hla_r

    def with_seed(self, seed: int) -> "HotOptions":
        """The same options under another stochastic-rounding key; reuses the built C struct."""
        seed = int(seed)
        if seed == self.seed:
            return self
        other = replace(self, seed=seed)
        base = self.to_c()
        c = _lib.HotConfig.from_buffer_copy(base)
        c.seed = seed & 0xFFFFFFFFFFFFFFFF
        object.__setattr__(other, "_c", c)
        object.__setattr__(other, "_keep", base)     # owner of what hla_rows_big points to
        return other

    def to_c(self) -> _lib.HotConfig:
        """struct hot_config for these options (built once per object; the library only reads it)."""
        c = self.__dict__.get("_c")
        if c is None:
            c = self._build_c()
            object.__setattr__(self, "_c", c)
        return c

    def _build_c(self) -> _lib.HotConfig:
        if self.hla_n > _lib.HOT_MAX_HLA_BIG:
            raise HotError("HLA block %d exceeds the native maximum %d" % (self.hla_n, _lib.HOT_MAX_HLA_BIG))
        c = _lib.HotConfig()
        c.n_o, c.hla_n, c.hla_r = self.n_o, self.hla_n, self.hla_r
        if self.hla_n > _lib.HOT_MAX_HLA_N:
            big = (C.c_int32 * self.hla_r)(*[int(v) for v in self.hla_rows])
            c.hla_rows_big = C.cast(big, C.POINTER(C.c_int32))
            c._rows_keepalive = big          # the struct only holds a pointer
        else:
            for i, v in enumerate(self.hla_rows):
                c.hla_rows[i] = int(v)
        c.gx_bits, c.w_bits, c.gw_bits, c.act_bits = self.gx_bits, self.w_bits, self.gw_bits, self.act_bits
        c.gx_round, c.w_round, c.gw_round, c.act_round = (_ROUND[self.gx_round], _ROUND[self.w_round],
                                                          _ROUND[self.gw_round], _ROUND[self.act_round])
        c.gx_scale, c.w_scale, c.gw_scale, c.act_scale = (_SCALE[self.gx_scale], _SCALE[self.w_scale],
                                                          _SCALE[self.gw_scale], _SCALE[self.act_scale])
        c.seed = int(self.seed) & 0xFFFFFFFFFFFFFFFF
        c.streams = int(self.streams)
        return c


def hq_rowwise(x: torch.Tensor, n: int = 16, bits: int = 4, rounding="nearest", scale="tensor",
               seed: int = 0, rng_stream: int = STREAM_GX) -> Tuple[torch.Tensor, torch.Tensor]:
    """Block-Hadamard along the last dim + absmax step + quantise.
    Returns (codes int8 [M, K*bits/8], steps fp32 [1] or [M])."""
    _need_gpu_2d(x, "input")
    M, K = x.shape
    mode = _SCALE[scale]
    codes = torch.empty((M, K * bits // 8), dtype=torch.int8, device=x.device)
    scales = torch.empty((M if mode == SCALE_ROW else 1,), dtype=torch.float32, device=x.device)
    ws = _ws(_lib.HOT_HQ_WORKSPACE_BYTES, x.device)
    _lib.check(_lib.lib().hot_hq_rowwise(x.data_ptr(), _dt(x), M, K, n, bits, _ROUND[rounding], seed, rng_stream,
                                         mode, codes.data_ptr(), scales.data_ptr(), ws.data_ptr(), ws.numel(),
                                         _stream()))
    return codes, scales


def hla_tokenwise(x: torch.Tensor, n: int, rows: Sequence[int], bits: int = 8, rounding="nearest",
                  scale="tensor", seed: int = 0, rng_stream: int = STREAM_GW, static_scratch: bool = False):
    """HLA along dim 0 + quantise, stored transposed.
    Returns (codes int8 [C, kpad(L')], steps fp32 [1] or [C], L').  With static_scratch the call goes
    through hot_hla_tokenwise_static: no workspace, the library's built-in scratch array."""
    _need_gpu_2d(x, "input")
    R, Cc = x.shape
    r = len(rows)
    kout = (R // max(n, 1)) * r
    ld = kpad(kout)
    mode = _SCALE[scale]
    codes = torch.empty((Cc, ld), dtype=torch.int8, device=x.device)
    scales = torch.empty((Cc if mode == SCALE_ROW else 1,), dtype=torch.float32, device=x.device)
    rows_c = (C.c_int32 * r)(*[int(v) for v in rows])
    if static_scratch:
        _lib.check(_lib.lib().hot_hla_tokenwise_static(x.data_ptr(), _dt(x), R, Cc, n, rows_c, r, bits,
                                                       _ROUND[rounding], seed, rng_stream, mode, codes.data_ptr(), ld,
                                                       scales.data_ptr(), _stream()))
        return codes, scales, kout
    ws = _ws(_lib.lib().hot_hla_workspace_bytes(R, Cc, n, r), x.device)
    _lib.check(_lib.lib().hot_hla_tokenwise(x.data_ptr(), _dt(x), R, Cc, n, rows_c, r, bits, _ROUND[rounding], seed,
                                            rng_stream, mode, codes.data_ptr(), ld, scales.data_ptr(),
                                            ws.data_ptr(), ws.numel(), _stream()))
    return codes, scales, kout


def wq_colwise(w: torch.Tensor, n: int = 16, bits: int = 4, rounding="nearest", scale="tensor",
               seed: int = 0, rng_stream: int = STREAM_W):
    """Block-Hadamard of W [O, I] along O + quantise, stored as [I, kpad(O)*bits/8]."""
    _need_gpu_2d(w, "W")
    O, I = w.shape
    ld = kpad(O) * bits // 8
    codes = torch.empty((I, ld), dtype=torch.int8, device=w.device)
    scales = torch.empty((1,), dtype=torch.float32, device=w.device)
    ws = _ws(_lib.lib().hot_colwise_workspace_bytes(I), w.device)
    _lib.check(_lib.lib().hot_wq_colwise(w.data_ptr(), _dt(w), O, I, n, bits, _ROUND[rounding], seed, rng_stream,
                                         _SCALE[scale], codes.data_ptr(), ld, scales.data_ptr(), ws.data_ptr(),
                                         ws.numel(), _stream()))
    return codes, scales


def gemm_plan(M: int, N: int, k: int, bits: int, lda: Optional[int] = None, ldb: Optional[int] = None,
              workspace_bytes: int = 0) -> int:
    """The kernel variant (enum hot_gemm_variant) the library runs for this product."""
    pitch = kpad(k) * bits // 8
    return int(_lib.lib().hot_gemm_plan(M, N, k, bits, lda or pitch, ldb or pitch, int(workspace_bytes)))


def gemm_i8(a: torch.Tensor, b: torch.Tensor, k: int, bits: int, scale_a: torch.Tensor, scale_b: torch.Tensor,
            post_scale: float = 1.0, out_dtype=torch.float32, return_acc: bool = False,
            variant: Optional[int] = None):
    """out[M,N] = ((A . B^T) * scale_a) * scale_b * post_scale on K-major codes.
    a [M, lda bytes], b [N, ldb bytes] int8 tensors whose rows hold k codes of
    `bits` bits, zero-padded to kpad(k).  `variant` (enum hot_gemm_variant) names the kernel
    (hot_gemm_i8_variant, with the workspace the variant asks for); None = hot_gemm_i8."""
    _need_gpu_2d(a, "A")
    _need_gpu_2d(b, "B")
    M, N = a.shape[0], b.shape[0]
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    acc = torch.empty((M, N), dtype=torch.int32, device=a.device) if return_acc else None
    per_row = 1 if scale_a.numel() > 1 else 0
    if per_row and scale_a.numel() != M:
        raise RuntimeError("scale_a must have 1 or M entries")
    if variant is None:
        _lib.check(_lib.lib().hot_gemm_i8(a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bits, M, N, k,
                                          scale_a.data_ptr(), per_row, scale_b.data_ptr(), float(post_scale),
                                          out.data_ptr(), _DTYPES[out_dtype], N,
                                          acc.data_ptr() if acc is not None else None, _stream()))
    else:
        need = int(_lib.lib().hot_gemm_workspace_bytes(M, N, k, bits))
        ws = _ws(need, a.device) if need else None
        _lib.check(_lib.lib().hot_gemm_i8_variant(a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bits, M, N, k,
                                                  scale_a.data_ptr(), per_row, scale_b.data_ptr(), float(post_scale),
                                                  out.data_ptr(), _DTYPES[out_dtype], N,
                                                  acc.data_ptr() if acc is not None else None, int(variant),
                                                  ws.data_ptr() if ws is not None else None,
                                                  ws.numel() if ws is not None else 0, _stream()))
    return (out, acc) if return_acc else out


def gemm_bf16(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None, out_dtype=torch.bfloat16,
              variant: int = 0) -> torch.Tensor:
    """out[M, N] = a[M, K] . b[N, K]^T (+ bias) on bf16 operands with fp32 accumulation (hot_gemm_bf16):
    F.linear(a, b, bias) through the data path of the integer kernels.  K a multiple of 128."""
    _need_gpu_2d(a, "A")
    _need_gpu_2d(b, "B")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise RuntimeError("gemm_bf16 takes bf16 operands")
    if a.stride(1) != 1 or b.stride(1) != 1 or a.shape[1] != b.shape[1]:
        raise RuntimeError("gemm_bf16 takes K-major operands of one K")
    M, K = a.shape
    N = b.shape[0]
    if bias is not None and (bias.dtype != out_dtype or bias.numel() != N or not bias.is_contiguous()):
        raise RuntimeError("bias must hold N contiguous elements of the output type")
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _lib.check(_lib.lib().hot_gemm_bf16(a.data_ptr(), a.stride(0) * 2, b.data_ptr(), b.stride(0) * 2, M, N, K,
                                        bias.data_ptr() if bias is not None else None, out.data_ptr(),
                                        _DTYPES[out_dtype], N, int(variant), _stream()))
    return out


def _launch_stream(side: Optional["torch.cuda.Stream"]) -> int:
    return _stream() if side is None else side.cuda_stream


class _on_stream:
    """Allocation context of a call whose kernels run on `side`: the outputs and the workspace are
    taken from the allocator UNDER that stream, so that they come from the side stream's own pool.  A
    block the current stream has just released (an operand copy of the GEMM that may still be running
    there) can then never be handed out and overwritten by the side stream's kernels."""

    def __init__(self, side):
        self.ctx = torch.cuda.stream(side) if side is not None else None

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def _join(side: Optional["torch.cuda.Stream"], *outputs: torch.Tensor) -> None:
    # the current stream waits for what `side` was given: enqueued before the call returns, which
    # orders every later use of the outputs on the current stream behind the kernels.  The outputs
    # belong to the side stream's pool; the allocator is told that the current stream uses them too.
    # (The workspace is released to the side stream's pool, whose next user is ordered behind the
    # kernels by that stream itself.)
    if side is not None:
        cur = torch.cuda.current_stream()
        cur.wait_stream(side)
        for t in outputs:
            t.record_stream(cur)


def abc_forward(x: torch.Tensor, opt: HotOptions, side: Optional["torch.cuda.Stream"] = None):
    """INT8 Hadamard-compressed activation buffer: (xq int8 [I, kpad(L')], sx fp32 [1]).
    With `side` the kernels run on that stream (which must already wait for x) beside whatever the
    current stream is doing, and the current stream joins it before the call returns."""
    _need_gpu_2d(x, "X")
    L, I = x.shape
    cfg = opt.to_c()
    with _on_stream(side):
        xq = torch.empty((I, kpad(opt.lprime(L))), dtype=torch.int8, device=x.device)
        sx = torch.empty((1,), dtype=torch.float32, device=x.device)
        ws = _ws(_lib.lib().hot_abc_workspace_bytes(L, I, C.byref(cfg)), x.device)
    try:
        _lib.check(_lib.lib().hot_abc_forward(x.data_ptr(), _dt(x), L, I, C.byref(cfg), xq.data_ptr(), sx.data_ptr(),
                                              ws.data_ptr(), ws.numel(), _launch_stream(side)))
    finally:
        _join(side, xq, sx)
    return xq, sx


def linear_backward(gy: torch.Tensor, w: torch.Tensor, xq: torch.Tensor, sx: torch.Tensor, opt: HotOptions,
                    out_dtype=None, timing: bool = False, workspace: Optional[torch.Tensor] = None,
                    bias_grad: bool = False):
    """g_x [L, I], g_W [O, I]; with timing=True also the four stage times (s), with
    timing="kernels" the eight per-kernel times of hot_linear_backward_kernels; with
    bias_grad=True also g_b [O], the sum of g_y over the tokens (hot_linear_backward_bias:
    delivered by the statistics pass, no extra read of g_y; not combined with timing)."""
    _need_gpu_2d(gy, "Go")
    _need_gpu_2d(w, "Wt")
    L, O = gy.shape
    if w.shape[0] != O:
        raise RuntimeError("W must be [O, I] with O = Go.shape[1]")
    if w.dtype != gy.dtype:
        raise RuntimeError("Go and W must have the same dtype")
    I = w.shape[1]
    out_dtype = out_dtype or gy.dtype
    cfg = opt.to_c()
    lp = opt.lprime(L)
    if tuple(xq.shape) != (I, kpad(lp)) or xq.dtype != torch.int8:
        raise RuntimeError("xq must be the int8 [I, kpad(L')] buffer written by abc_forward")
    sizes = opt.__dict__.setdefault("_ws_bytes", {})      # per options object: the query is a pure function of these
    need = sizes.get((L, O, I))
    if need is None:
        need = _lib.lib().hot_backward_workspace_bytes(L, O, I, C.byref(cfg))
        if need == 0:
            raise HotError("bad configuration: %s" % _lib.lib().hot_last_error().decode())
        sizes[(L, O, I)] = need
    if workspace is None or workspace.numel() < need:
        workspace = _ws(need, gy.device)
    gx = torch.empty((L, I), dtype=out_dtype, device=gy.device)
    gw = torch.empty((O, I), dtype=out_dtype, device=gy.device)
    if bias_grad:
        if timing:
            raise ValueError("bias_grad and timing are separate entry points")
        gb = torch.empty((O,), dtype=out_dtype, device=gy.device)
        _lib.check(_lib.lib().hot_linear_backward_bias(
            gy.data_ptr(), w.data_ptr(), _dt(gy), xq.data_ptr(), sx.data_ptr(), L, O, I, C.byref(cfg), gx.data_ptr(),
            gw.data_ptr(), gb.data_ptr(), _DTYPES[out_dtype], workspace.data_ptr(), workspace.numel(), _stream()))
        return gx, gw, gb
    per_kernel = timing == "kernels"
    times = (C.c_float * (8 if per_kernel else 4))() if timing else None
    entry = _lib.lib().hot_linear_backward_kernels if per_kernel else _lib.lib().hot_linear_backward
    _lib.check(entry(gy.data_ptr(), w.data_ptr(), _dt(gy), xq.data_ptr(), sx.data_ptr(), L, O, I, C.byref(cfg),
                     gx.data_ptr(), gw.data_ptr(), _DTYPES[out_dtype], workspace.data_ptr(), workspace.numel(),
                     times, _stream()))
    if timing:
        return gx, gw, [float(t) for t in times]
    return gx, gw


def backward_streams(L: int, O: int, I: int, opt: HotOptions) -> int:
    """1 or 2: the launch order linear_backward takes for this shape (hot_backward_streams)."""
    return int(_lib.lib().hot_backward_streams(int(L), int(O), int(I), C.byref(opt.to_c())))


def kpad_group(T: int, opt: HotOptions) -> int:
    """Code bytes every sample takes in the K dimension of the batched g_W operands."""
    return int(_lib.lib().hot_kpad_group(int(T), C.byref(opt.to_c())))


def backward_batched_ranges(B: int, T: int, O: int, I: int, opt: HotOptions) -> int:
    """Ranges of consecutive samples in which linear_backward_batched adds up the weight gradient
    (hot_backward_batched_ranges): each range in sample order, then the range sums in order."""
    return int(_lib.lib().hot_backward_batched_ranges(int(B), int(T), int(O), int(I), C.byref(opt.to_c())))


def abc_forward_batched(x: torch.Tensor, opt: HotOptions, side: Optional["torch.cuda.Stream"] = None):
    """Activation buffer of a 3-D input [B, T, I] with one step per sample (hot_abc_forward_batched):
    (xq int8 [I, B * kpad_group(T)], sx fp32 [B]).  `side`: as in abc_forward."""
    if not x.is_cuda or x.dim() != 3 or not x.is_contiguous():
        raise RuntimeError("X must be a contiguous CUDA tensor [B, T, I]!")
    B, T, I = x.shape
    cfg = opt.to_c()
    kg = kpad_group(T, opt)
    with _on_stream(side):
        xq = torch.empty((I, B * kg), dtype=torch.int8, device=x.device)
        sx = torch.empty((B,), dtype=torch.float32, device=x.device)
        ws = _ws(_lib.lib().hot_abc_batched_workspace_bytes(B, T, I, C.byref(cfg)), x.device)
    try:
        _lib.check(_lib.lib().hot_abc_forward_batched(x.data_ptr(), _dt(x), B, T, I, C.byref(cfg), xq.data_ptr(),
                                                      sx.data_ptr(), ws.data_ptr(), ws.numel(), _launch_stream(side)))
    finally:
        _join(side, xq, sx)
    return xq, sx


def linear_backward_batched(gy: torch.Tensor, w: torch.Tensor, xq: torch.Tensor, sx: torch.Tensor, opt: HotOptions,
                            out_dtype=None, workspace: Optional[torch.Tensor] = None):
    """g_x [B, T, I] and g_W [O, I] (summed over the samples) for g_y [B, T, O] with one set of steps per
    sample (hot_linear_backward_batched)."""
    if not gy.is_cuda or gy.dim() != 3 or not gy.is_contiguous():
        raise RuntimeError("Go must be a contiguous CUDA tensor [B, T, O]!")
    _need_gpu_2d(w, "Wt")
    B, T, O = gy.shape
    if w.shape[0] != O or w.dtype != gy.dtype:
        raise RuntimeError("W must be [O, I] with O = Go.shape[2], in the dtype of Go")
    I = w.shape[1]
    out_dtype = out_dtype or gy.dtype
    cfg = opt.to_c()
    kg = kpad_group(T, opt)
    if tuple(xq.shape) != (I, B * kg) or xq.dtype != torch.int8 or sx.numel() != B:
        raise RuntimeError("xq / sx must be the buffers written by abc_forward_batched")
    need = _lib.lib().hot_backward_batched_workspace_bytes(B, T, O, I, C.byref(cfg))
    if need == 0:
        raise HotError("bad configuration: %s" % _lib.lib().hot_last_error().decode())
    if workspace is None or workspace.numel() < need:
        workspace = _ws(need, gy.device)
    gx = torch.empty((B, T, I), dtype=out_dtype, device=gy.device)
    gw = torch.empty((O, I), dtype=out_dtype, device=gy.device)
    _lib.check(_lib.lib().hot_linear_backward_batched(gy.data_ptr(), w.data_ptr(), _dt(gy), xq.data_ptr(), sx.data_ptr(), B, T,
                                                      O, I, C.byref(cfg), gx.data_ptr(), gw.data_ptr(), _DTYPES[out_dtype],
                                                      workspace.data_ptr(), workspace.numel(), _stream()))
    return gx, gw


def gx_lowrank(gy: torch.Tensor, w: torch.Tensor, opt: HotOptions, out_dtype=None) -> torch.Tensor:
    """g_x [L, I] of the schemes "low_rank" / "gilr_gwh" (hot_gx_lowrank): P^T (q(P g_y) q(W)) s_g s_w / n with
    W untransformed; opt.hla_n / hla_rows describe P, gx_* the quantiser of P g_y, w_* that of W."""
    _need_gpu_2d(gy, "Go")
    _need_gpu_2d(w, "Wt")
    L, O = gy.shape
    if w.shape[0] != O or w.dtype != gy.dtype:
        raise RuntimeError("W must be [O, I] with O = Go.shape[1], in the dtype of Go")
    I = w.shape[1]
    out_dtype = out_dtype or gy.dtype
    cfg = opt.to_c()
    need = _lib.lib().hot_gx_lowrank_workspace_bytes(L, O, I, C.byref(cfg))
    if need == 0:
        raise HotError("bad configuration: %s" % _lib.lib().hot_last_error().decode())
    ws = _ws(need, gy.device)
    gx = torch.empty((L, I), dtype=out_dtype, device=gy.device)
    _lib.check(_lib.lib().hot_gx_lowrank(gy.data_ptr(), w.data_ptr(), _dt(gy), L, O, I, C.byref(cfg), gx.data_ptr(),
                                         _DTYPES[out_dtype], ws.data_ptr(), ws.numel(), _stream()))
    return gx


def gx_luq(gy: torch.Tensor, w: torch.Tensor, opt: HotOptions, out_dtype=None) -> torch.Tensor:
    """g_x [L, I] with the logarithmic quantiser on g_y (hot_gx_luq; quantBWDGogi = "luq"): opt.n_o, the 4-bit
    widths, opt.w_round / w_scale for W and opt.seed are read."""
    _need_gpu_2d(gy, "Go")
    _need_gpu_2d(w, "Wt")
    L, O = gy.shape
    if w.shape[0] != O or w.dtype != gy.dtype:
        raise RuntimeError("W must be [O, I] with O = Go.shape[1], in the dtype of Go")
    I = w.shape[1]
    out_dtype = out_dtype or gy.dtype
    cfg = opt.to_c()
    need = _lib.lib().hot_gx_luq_workspace_bytes(L, O, I, C.byref(cfg))
    if need == 0:
        raise HotError("bad configuration: %s" % _lib.lib().hot_last_error().decode())
    ws = _ws(need, gy.device)
    gx = torch.empty((L, I), dtype=out_dtype, device=gy.device)
    _lib.check(_lib.lib().hot_gx_luq(gy.data_ptr(), w.data_ptr(), _dt(gy), L, O, I, C.byref(cfg), gx.data_ptr(),
                                     _DTYPES[out_dtype], ws.data_ptr(), ws.numel(), _stream()))
    return gx


def gw_luq(gy: torch.Tensor, xq: torch.Tensor, sx: torch.Tensor, opt: HotOptions, out_dtype=None) -> torch.Tensor:
    """g_W [O, I] with the logarithmic quantiser on the projected g_y (hot_gw_luq; quantBWDGogw = "luq" or
    luq_quantizer picked for g_W under quantAuto): opt.hla_n / hla_rows, gw_bits = 4 and opt.seed are read;
    xq [I, kpad(L')] / sx [1] as abc_forward writes them."""
    _need_gpu_2d(gy, "Go")
    _need_gpu_2d(xq, "xq")
    L, O = gy.shape
    I = xq.shape[0]
    lp = (L // opt.hla_n) * opt.hla_r
    if xq.dtype != torch.int8 or xq.stride(0) != kpad(lp) or xq.stride(1) != 1:
        raise RuntimeError("xq must be the [I, kpad(L')] INT8 buffer of abc_forward")
    out_dtype = out_dtype or gy.dtype
    cfg = opt.to_c()
    need = _lib.lib().hot_gw_luq_workspace_bytes(L, O, I, C.byref(cfg))
    if need == 0:
        raise HotError("bad configuration: %s" % _lib.lib().hot_last_error().decode())
    ws = _ws(need, gy.device)
    gw = torch.empty((O, I), dtype=out_dtype, device=gy.device)
    _lib.check(_lib.lib().hot_gw_luq(gy.data_ptr(), _dt(gy), xq.data_ptr(), sx.data_ptr(), L, O, I, C.byref(cfg),
                                     gw.data_ptr(), _DTYPES[out_dtype], ws.data_ptr(), ws.numel(), _stream()))
    return gw


def measure_ceilings(device=None):
    """(copy GB/s, INT8 MFMA TOP/s) of this box from the library's two plain ceiling kernels."""
    device = device or torch.device("cuda", torch.cuda.current_device())
    buf = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    copy, mfma = C.c_float(0), C.c_float(0)
    _lib.check(_lib.lib().hot_measure_ceilings(buf.data_ptr(), buf.numel(), C.byref(copy), C.byref(mfma), _stream()))
    return float(copy.value), float(mfma.value)
