"""Host-side logic of the package (no GPU): helper API with the reference's
names, option mapping, the C-ABI library's exports and its argument checks."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

from oracle import hot_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ----------------------------------------------------------- helper surface

def test_helpers_agree_with_oracle():
    from hot_amd import hadamard_matmul as hm
    for size in (1, 2, 4, 12, 16, 48, 49, 64, 197, 768, 3072, 11008, 12608, 25216):
        assert hm.biggest_power2_factor(size) == orc.pow2_factor(size)
        assert hm.biggest_power2_factor_max16(size) == orc.pow2_factor_max16(size)
        assert np.array_equal(hm.make_hadamard(size), orc.make_hadamard(size))
        n, rows = hm.hla_rows(size)
        n2, rows2 = orc.hla_rows(size)
        assert n == n2 and np.array_equal(rows, rows2)
        if n <= 256:
            assert np.array_equal(hm.make_WHT(size), orc.make_WHT(size))
    assert hm.make_WHT(8192).shape == (2080, 8192)
    n, rows = hm.paper_rows(16, 8)
    assert np.array_equal(rows, orc.paper_rows(16, 8)[1])
    with pytest.raises(ValueError):
        hm.hadamard(12)


def test_lowering_matmuls():
    from hot_amd import hadamard_matmul as hm
    rng = np.random.default_rng(0)
    a = rng.integers(-20, 20, (128, 48)).astype(np.float32)
    H = torch.tensor(hm.hadamard(16), dtype=torch.float32)
    assert np.array_equal(hm.lowering_matmul_front(torch.from_numpy(a), H).numpy(), orc.fwht_blocks_last(a, 16))
    assert np.array_equal(hm.lowering_matmul_back(H, torch.from_numpy(a)).numpy(), orc.fwht_blocks_first(a, 16))
    P = torch.tensor(hm.make_WHT(64), dtype=torch.float32)
    n, rows = orc.hla_rows(64)
    assert np.array_equal(hm.lowering_matmul_back(P, torch.from_numpy(a)).numpy(), orc.fwht_blocks_first(a, n, rows))
    a3 = torch.from_numpy(np.stack([a, 2 * a]))
    assert hm.lowering_matmul_back(P, a3).shape == (2, 72, 48)
    assert np.array_equal(hm.lowering_matmul_front(a3, H)[1].numpy(), orc.fwht_blocks_last(2 * a, 16))
    # whole-dimension case: plain matmul
    assert np.array_equal(hm.lowering_matmul_back(torch.tensor(hm.make_WHT(128), dtype=torch.float32),
                                                  torch.from_numpy(a)).numpy(),
                          orc.fwht_blocks_first(a, 128, orc.hla_rows(128)[1]))


def test_transform_dict_caches():
    from hot_amd.hadamard_matmul import Transform_Dict
    td = Transform_Dict()
    h = td.get_or_register("hadamard", 3072)
    assert h.shape == (16, 16) and td.get_or_register("hadamard", 3072) is h
    assert td.get_or_register("low_rank", 12608, 50).shape == (36, 64)
    with pytest.raises(NotImplementedError):
        td.get_or_register("haar", 8)


# ------------------------------------------------------------ option mapping

@pytest.fixture
def fresh_args():
    from hot_amd import args
    saved = {k: getattr(args, k) for k in dir(args) if not k.startswith("_")}
    args.hot_recipe()          # the module defaults describe a plain layer, as the reference's do
    yield args
    for k, v in saved.items():
        setattr(args, k, v)


def test_options_follow_args(fresh_args):
    from hot_amd import ops
    from hot_amd.quant_matmul import options_for
    a = fresh_args
    o = options_for(12608)
    assert (o.hla_n, o.hla_r, o.n_o) == (64, 36, 16)
    assert (o.gx_bits, o.w_bits, o.gw_bits, o.act_bits) == (4, 4, 8, 8)
    assert o.gx_round == ops.ROUND_NEAREST and o.gx_scale == ops.SCALE_TENSOR
    a.quantBWDGogi, a.quantBWDWgt, a.quantBWDGogw, a.quantBWDAct = "nq", "sawb", "stoch", "sawb"
    o = options_for(12608)
    assert (o.gx_round, o.gx_scale) == (ops.ROUND_STOCH, ops.SCALE_ROW)
    assert (o.w_round, o.w_scale) == (ops.ROUND_NEAREST, ops.SCALE_SAWB)
    assert (o.gw_round, o.gw_scale) == (ops.ROUND_STOCH, ops.SCALE_TENSOR)
    assert o.act_scale == ops.SCALE_SAWB
    # layer-wise selection: the g_W branch reads the g_x bit width (utils/quant_matmul.py:308)
    a.quantAuto = True
    a.layer_quant_dict["blk_gx"] = "norm_quantizer"
    a.layer_quant_dict["blk_gw"] = "stoch_quantizer"
    o = options_for(12608, "blk")
    assert (o.gx_scale, o.gw_scale, o.gw_bits) == (ops.SCALE_ROW, ops.SCALE_TENSOR, 4)
    a.layer_quant_dict.clear()
    a.quantAuto = False
    # token rules
    assert options_for(197).hla_n == 1
    o = options_for(8192)                           # the reference's rule, whatever the block size
    assert (o.hla_n, o.hla_r) == (8192, 2080)
    a.hla_max_block = 64
    o = options_for(8192)
    assert (o.hla_n, o.hla_r) == (64, 36)
    a.hla_max_block = 8192
    a.hla_rule = "paper"
    o = options_for(8192)
    assert (o.hla_n, o.hla_r) == (16, 8)
    a.hla_rule = "python"
    a.quantBWDGogi = "luq"                          # an entry point of its own for the g_x product
    from hot_amd.quant_matmul import gx_uses_luq
    assert gx_uses_luq() and options_for(64).gx_bits == 4
    a.quantBWDGogw = "luq"                          # and one for the g_W product
    from hot_amd.quant_matmul import gw_uses_luq
    assert gw_uses_luq() and options_for(64).gw_round == ops.ROUND_STOCH
    a.quantBWDGogw = "int"
    assert not gw_uses_luq()
    a.quantBWDGogi = "int"
    assert not gx_uses_luq()
    a.transform_scheme = "hadamard"                 # block Hadamard along the tokens, nothing dropped
    o = options_for(12608)
    assert (o.hla_n, o.hla_r, o.hla_rows) == (16, 16, tuple(range(16)))
    assert options_for(197).hla_n == 1 and options_for(200).hla_n == 8
    a.transform_scheme = "low_rank"                 # g_W side as gih_gwlr; the g_x side has a rule of its own
    from hot_amd.quant_matmul import gx_token_rule
    o = options_for(12608)
    assert (o.hla_n, o.hla_r) == (64, 36)
    assert gx_token_rule(8192)[0] == 8192 and len(gx_token_rule(8192)[1]) == 2080    # the reference's own rule
    assert gx_token_rule(25216)[0] == 128 and len(gx_token_rule(25216)[1]) == 36
    a.hla_max_block = 64
    assert gx_token_rule(8192)[0] == 64 and len(gx_token_rule(8192)[1]) == 36
    a.hla_max_block = 8192
    a.transform_scheme = "gilr_gwh"                 # g_W side as hadamard
    o = options_for(12608)
    assert (o.hla_n, o.hla_r) == (16, 16)
    assert gx_token_rule(12608)[0] == 64
    a.transform_scheme = "gilro_gwh"
    with pytest.raises(NotImplementedError):
        options_for(64)
    a.transform_scheme = "gih_gwlr"
    a.TransformInput = False
    with pytest.raises(NotImplementedError):
        options_for(64)


def test_hq_linear_surface_and_no_cpu_fallback(fresh_args):
    import torch.nn as nn
    from hot_amd.quant_matmul import FLinearQ, HQ_Linear
    lin = HQ_Linear(48, 64)
    assert isinstance(lin, nn.Linear) and lin.hadamard_out.shape == (16, 16) and lin.layer_name == " "
    assert "hadamard_out" not in lin.state_dict() and "hadamard_bs" not in lin.state_dict()
    assert {"forward", "setup_context", "backward"} <= set(vars(FLinearQ))
    with pytest.raises(RuntimeError):           # the native path refuses CPU tensors, it never falls back
        lin(torch.randn(128, 48))
    # the module defaults are the reference's: a plain full-precision layer, which runs anywhere
    fresh_args.plain_recipe()
    x = torch.randn(128, 48, requires_grad=True)
    lin(x).sum().backward()
    assert x.grad is not None and lin.weight.grad.shape == (64, 48)


def test_args_defaults_are_the_reference_defaults():
    """args.py:29-49 of the reference: widths 0, quantisers "no", transforms off, scheme gih_gwlr."""
    import importlib
    from hot_amd import args
    fresh = importlib.reload(args)
    try:
        assert (fresh.GogiQuantBit, fresh.weightQuantBit, fresh.GogwQuantBit, fresh.actQuantBit) == (0, 0, 0, 0)
        assert (fresh.quantBWDGogi, fresh.quantBWDWgt, fresh.quantBWDGogw, fresh.quantBWDAct) == ("no",) * 4
        assert not (fresh.TransformGogi or fresh.TransformWgt or fresh.TransformGogw or fresh.TransformInput)
        assert fresh.transform_scheme == "gih_gwlr" and fresh.quantAuto is False and fresh.eps == 1e-11
        fresh.canonical_recipe()
        assert (fresh.quantBWDGogi, fresh.quantBWDWgt, fresh.quantBWDGogw, fresh.quantBWDAct) == ("nq", "sawb", "nq", "sawb")
        assert (fresh.GogiQuantBit, fresh.weightQuantBit, fresh.GogwQuantBit, fresh.actQuantBit) == (4, 4, 8, 8)
        assert fresh.quantAuto and fresh.TransformGogi and fresh.TransformInput
    finally:
        fresh.plain_recipe()


def test_replace_layers_style_surgery():
    """The reference swaps layers by constructing new(in_features, out_features)
    and re-pointing weight/bias data (utils/utils.py:53-74)."""
    import torch.nn as nn
    from hot_amd.quant_matmul import HQ_Linear
    model = nn.Sequential(nn.Linear(32, 64), nn.GELU(), nn.Linear(64, 16))
    for name, mod in list(model.named_children()):
        if isinstance(mod, nn.Linear):
            new = HQ_Linear(mod.in_features, mod.out_features)
            new.weight.data = mod.weight.data
            new.bias.data = mod.bias.data
            setattr(model, name, new)
    assert isinstance(model[0], HQ_Linear) and model[2].weight.shape == (16, 64)


def test_hlq_backward_checks_like_the_reference():
    from hot_amd import HLQ_backward
    z = torch.zeros(4, 16)
    with pytest.raises(RuntimeError, match="Go must be a CUDA tensor!"):
        HLQ_backward.backward(z, z, z, 0, 0, 16, True)


# --------------------------------------------------------------- the C ABI

def _declared():
    text = open(os.path.join(ROOT, "include", "hot_gfx950.h")).read()
    return re.findall(r"HOT_API\s+[\w\s\*]+?\b(hot_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    from hot_amd import _lib
    names = _declared()
    assert len(names) >= 12 and set(names) == set(_lib.EXPORTS)
    lib = C.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert _lib.lib().hot_abi_version() == 4
    header = open(os.path.join(ROOT, "include", "hot_gfx950.h")).read()
    for name in ("HOT_MAX_HLA_N", "HOT_MAX_HLA_BIG", "HOT_HQ_WORKSPACE_BYTES", "HOT_STATIC_MAX_CHANNELS"):   # the binding repeats these constants
        assert int(re.search(r"#define\s+%s\s+(\d+)" % name, header).group(1)) == getattr(_lib, name)
    enum = re.search(r"enum hot_gemm_variant \{(.*?)\};", header, re.S).group(1)
    for name, val in re.findall(r"HOT_(GEMM_\w+)\s*=\s*(\d+)", enum):
        if name != "GEMM_VARIANTS":
            assert getattr(_lib, name) == int(val), name
    assert [_lib.lib().hot_kpad(k) for k in (1, 128, 129, 7092)] == [128, 128, 256, 7168]


def test_library_argument_checks_need_no_gpu():
    from hot_amd import _lib, ops
    lib = _lib.lib()
    one = C.c_void_p(4096)  # never dereferenced: every call below fails validation first
    assert lib.hot_hq_rowwise(one, 0, 4, 64, 12, 4, 0, 0, 0, 0, one, one, None, 0, None) == -2
    assert b"Hadamard block" in lib.hot_last_error()
    assert lib.hot_hq_rowwise(one, 0, 4, 40, 16, 4, 0, 0, 0, 0, one, one, None, 0, None) == -1
    assert lib.hot_hq_rowwise(one, 0, 4, 64, 16, 4, 0, 0, 0, 0, one, one, None, 0, None) == -3   # no workspace
    assert lib.hot_gemm_i8(one, 64, one, 64, 8, 4, 4, 100, one, 0, one, 1.0, one, 0, 4, None, None) == -1
    assert b"row pitches" in lib.hot_last_error()
    rows = (C.c_int32 * 2)(0, 0)
    assert lib.hot_hla_tokenwise(one, 0, 64, 8, 16, rows, 2, 8, 0, 0, 0, 0, one, 128, one, one, 1 << 30, None) == -1
    assert b"listed twice" in lib.hot_last_error()
    # the variant query and the named-variant entry point validate before they touch anything
    assert lib.hot_gemm_plan(12608, 768, 3072, 4, 1536, 1536, 0) == _lib.GEMM_SLOT_160X256
    assert lib.hot_gemm_plan(12608, 768, 2304, 4, 1152, 1152, 0) == _lib.GEMM_DMA_128_S3
    # INT8 products with room to spare at 128 x 128 take the shortest tile that keeps one round (ViT-B g_W products)
    assert lib.hot_gemm_plan(3072, 768, 7092, 8, 7168, 7168, 0) == _lib.GEMM_SLOT_96X128        # fc1: 192 tiles
    assert lib.hot_gemm_plan(3072, 768, 7092, 8, 7168, 7168, 1 << 30) == _lib.GEMM_SLOT_96X128  # a workspace changes nothing
    assert lib.hot_gemm_plan(2304, 768, 7092, 8, 7168, 7168, 0) == _lib.GEMM_SLOT_64X128        # qkv: 216 tiles
    assert lib.hot_gemm_plan(768, 768, 7092, 8, 7168, 7168, 1 << 30) == _lib.GEMM_SLOT_32X128   # proj: 144 tiles, no split
    assert lib.hot_gemm_plan(768, 3072, 7092, 8, 7168, 7168, 0) == _lib.GEMM_SLOT_96X128        # fc2: 192 tiles
    assert lib.hot_gemm_plan(4096, 1024, 7092, 8, 7168, 7168, 0) == _lib.GEMM_SLOT_128          # 256 tiles: nothing shorter fits
    assert lib.hot_gemm_plan(768, 768, 7092, 4, 3584, 3584, 1 << 30) == _lib.GEMM_DMA_128_SPLITK # INT4: 36 tiles, split K
    assert lib.hot_gemm_plan(8192, 4096, 11008, 4, 5504, 5504, 0) == _lib.GEMM_SLOT_256
    assert lib.hot_gemm_plan(8192, 4096, 11136, 4, 5568, 5568, 0) == _lib.GEMM_DMA_256_S4     # rows of 43.5 lines
    assert lib.hot_gemm_plan(1 << 20, 128, 8192, 8, 8192, 8192, 0) == _lib.GEMM_REG_128     # A is 8 GiB
    assert lib.hot_gemm_workspace_bytes(3072, 768, 7092, 8) == 144 * 3 * 128 * 128 * 4      # what the split-K variant would take
    assert lib.hot_gemm_i8_variant(one, 128, one, 128, 8, 4, 4, 100, one, 0, one, 1.0, one, 0, 4, None, 99, None, 0, None) == -1
    assert b"variant" in lib.hot_last_error()
    assert lib.hot_gemm_i8_variant(one, 128, one, 128, 8, 4, 4, 100, one, 0, one, 1.0, one, 0, 4, None,
                                   _lib.GEMM_DMA_128_SPLITK, None, 0, None) == -2      # nothing to split
    # the entry point without a workspace: limits checked before anything else
    assert lib.hot_hla_tokenwise_static(one, 0, 512, 64, 256, rows, 2, 8, 0, 0, 0, 0, one, 128, one, None) == -2
    assert lib.hot_hla_tokenwise_static(one, 0, 64, _lib.HOT_STATIC_MAX_CHANNELS + 8, 16, rows, 2, 8, 0, 0, 0, 0, one, 128, one, None) == -2
    assert b"channels exceed" in lib.hot_last_error()
    cfg = ops.HotOptions(hla_n=64, hla_rows=tuple(range(36))).to_c()
    need = lib.hot_backward_workspace_bytes(12608, 3072, 768, C.byref(cfg))
    # packed g_y codes + packed W codes + int8 low-rank g_y codes dominate
    assert need >= 12608 * 1536 + 768 * 1536 + 3072 * 7168
    cfg.n_o = 12            # not a power of two
    assert lib.hot_backward_workspace_bytes(12608, 3072, 768, C.byref(cfg)) == 0
    with pytest.raises(_lib.HotError):
        _lib.check(-2)


def test_bench_refuses_more_than_one_gpu():
    """Every box has one GPU: the benchmark says so instead of running a second rank."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
