"""Seeded random shapes and settings through the four backward entry points against the oracle: the
fixed cases of test_gpu_backward.py name the corners, these walk the space between them (block sizes
1 ... 128, ragged strips, every quantiser variant, both dtypes).  Bit-exact, like the fixed cases."""
import random

import numpy as np
import pytest
import torch

from oracle import hot_oracle as orc
from test_gpu_backward import make_case, run_both

pytestmark = pytest.mark.gpu

VARIANTS = [
    dict(), dict(gx_bits=8, w_bits=8), dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW),
    dict(gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, act_round=orc.ROUND_STOCH, seed=5),
    dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH, gw_scale=orc.SCALE_ROW, seed=11),
    dict(w_scale=orc.SCALE_SAWB, act_scale=orc.SCALE_SAWB),
    dict(gx_round=orc.ROUND_STOCH, w_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, seed=3),
]


def _options(ocfg):
    from hot_amd import ops
    return ops.HotOptions(n_o=ocfg.n_o, hla_n=ocfg.hla_n, hla_rows=ocfg.hla_rows, gx_bits=ocfg.gx_bits, w_bits=ocfg.w_bits,
                          gw_bits=ocfg.gw_bits, act_bits=ocfg.act_bits, gx_round=ocfg.gx_round, w_round=ocfg.w_round,
                          gw_round=ocfg.gw_round, act_round=ocfg.act_round, gx_scale=ocfg.gx_scale, w_scale=ocfg.w_scale,
                          gw_scale=ocfg.gw_scale, act_scale=ocfg.act_scale, seed=ocfg.seed)


def _widths(rnd):
    return 16 * rnd.choice([1, 2, 3, 5, 8, 13, 16, 17, 24]), 8 * rnd.choice([1, 2, 3, 5, 9, 16, 20, 33])


@pytest.mark.parametrize("case", range(10))
def test_random_flat_backward(gpu, case):
    rnd = random.Random(1000 + case)
    n = rnd.choice([1, 2, 4, 8, 16, 32, 64, 128])
    L = n * rnd.choice([1, 3, 5, 7, 9, 13, 21])
    if L < 16:
        L = 16 * (L // n)
    O, I = _widths(rnd)
    dt = rnd.choice([torch.float32, torch.bfloat16])
    x, w, gy = make_case(L, O, I, seed=case, dtype=dt)
    ocfg = orc.HotConfig.python_rule(L, **rnd.choice(VARIANTS))
    gx, gw, tr = run_both(x, w, gy, ocfg, _options(ocfg), gpu)
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dt)) and torch.equal(gw.cpu(), torch.from_numpy(tr.g_w).to(dt))


@pytest.mark.parametrize("case", range(10))
def test_random_batched_backward(gpu, case):
    from hot_amd import ops
    rnd = random.Random(2000 + case)
    B = rnd.choice([1, 2, 3, 5, 8, 17, 40])
    T = rnd.choice([1, 2, 4, 8, 16, 32, 64, 128]) * rnd.choice([1, 3, 5]) if rnd.random() < 0.7 else rnd.choice([197, 49, 50, 77, 196])
    O, I = _widths(rnd)
    dt = rnd.choice([torch.float32, torch.bfloat16])
    g = torch.Generator().manual_seed(case)
    mag = 10.0 ** (torch.rand(B, 1, 1, generator=g) * 3 - 3)
    x = (torch.randn(B, T, I, generator=g) * (mag * 100)).to(dt)
    w = ((torch.rand(O, I, generator=g) * 2 - 1) / I ** 0.5).to(dt)
    gy = (torch.randn(B, T, O, generator=g) * mag).to(dt)
    ocfg = orc.HotConfig.python_rule(T, **rnd.choice(VARIANTS))
    opt = _options(ocfg)
    xq, sx = ops.abc_forward_batched(x.to(gpu), opt)
    gx, gw = ops.linear_backward_batched(gy.to(gpu), w.to(gpu), xq, sx, opt)
    xq_ref, sx_ref = orc.abc_forward_batched(x.float().numpy(), ocfg)
    ranges = ops.backward_batched_ranges(B, T, O, I, opt)
    gx_ref, gw_ref, _ = orc.linear_backward_batched(gy.float().numpy(), w.float().numpy(), xq_ref, sx_ref, ocfg, gw_ranges=ranges)
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    assert torch.equal(gx.cpu(), torch.from_numpy(gx_ref).to(dt)) and torch.equal(gw.cpu(), torch.from_numpy(gw_ref).to(dt))


@pytest.mark.parametrize("case", range(8))
def test_random_lowrank_gx(gpu, case):
    from hot_amd import ops
    rnd = random.Random(3000 + case)
    n = rnd.choice([1, 2, 4, 8, 16, 32, 64])
    L = n * rnd.choice([1, 3, 5, 7, 9, 13, 21])
    if L < 16:
        L = 16 * (L // n)
    O, I = _widths(rnd)
    dt = rnd.choice([torch.float32, torch.bfloat16])
    v = {k: val for k, val in rnd.choice(VARIANTS).items() if k in ("gx_bits", "w_bits", "gx_round", "w_round", "w_scale", "seed")}
    ocfg = orc.HotConfig.python_rule(L, **v)
    x, w, gy = make_case(L, O, I, seed=case, dtype=dt)
    gx = ops.gx_lowrank(gy.to(gpu), w.to(gpu), _options(ocfg))
    tr = orc.gx_lowrank(gy.float().numpy(), w.float().numpy(), ocfg)
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dt))


@pytest.mark.parametrize("case", range(8))
def test_random_luq_gx(gpu, case):
    from hot_amd import ops
    rnd = random.Random(4000 + case)
    L = rnd.choice([1, 7, 49, 197, 448, 1000, 2048])
    O, I = _widths(rnd)
    dt = rnd.choice([torch.float32, torch.bfloat16])
    ocfg = orc.HotConfig(seed=case, w_round=rnd.choice([orc.ROUND_NEAREST, orc.ROUND_STOCH]),
                         w_scale=rnd.choice([orc.SCALE_TENSOR, orc.SCALE_SAWB]))
    x, w, gy = make_case(L, O, I, seed=case, dtype=dt)
    opt = ops.HotOptions(n_o=ocfg.n_o, w_round=ocfg.w_round, w_scale=ocfg.w_scale, seed=ocfg.seed)
    gx = ops.gx_luq(gy.to(gpu), w.to(gpu), opt)
    tr = orc.gx_luq(gy.float().numpy(), w.float().numpy(), ocfg)
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dt))
