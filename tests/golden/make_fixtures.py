"""Writes the fixtures of this folder from the CPU oracle (oracle/hot_oracle.py).

They are snapshots of the ORACLE's canonical semantics, not outputs of the reference (which ships no
vectors for this path and was not run): they pin the oracle against drift — a change of a summation
order, of the RNG numbering or of a rounding rule changes a fixture — and give the GPU tests a second,
frozen target.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import hot_oracle as orc  # noqa: E402


def case(data_seed, L, O, I, **kw):
    rng = np.random.default_rng(data_seed)
    x = rng.standard_normal((L, I)).astype(np.float32)
    w = (rng.uniform(-1, 1, (O, I)) / np.sqrt(I)).astype(np.float32)
    gy = (rng.standard_normal((L, O)) * 1e-3).astype(np.float32)
    gy[rng.uniform(size=gy.shape) < 0.01] *= 50
    cfg = orc.HotConfig.python_rule(L, **kw)
    xq, sx = orc.abc_forward(x, cfg)
    tr = orc.linear_backward(gy, w, xq, sx, cfg)
    return dict(x=x, w=w, gy=gy, hla_n=np.int32(cfg.hla_n), hla_rows=np.asarray(cfg.hla_rows, np.int32),
                xq=xq, sx=sx, qG=tr.qG, sG=tr.sG, qW=tr.qW, sW=tr.sW, qGp=tr.qGp, sGp=tr.sGp,
                acc_x=tr.acc_x, acc_w=tr.acc_w, g_x=tr.g_x, g_w=tr.g_w)


CASES = {
    # name: (data seed, L, O, I, HotConfig overrides; `seed` there keys the stochastic rounding)
    "nearest_int4_L320_O64_I48": (0, 320, 64, 48, {}),
    "stoch_row_int8_L192_O32_I40": (1, 192, 32, 40, dict(gx_bits=8, w_bits=8, gx_round=orc.ROUND_STOCH,
                                                         gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
                                                         gw_scale=orc.SCALE_ROW, seed=1234)),
}


def main():
    for name, (data_seed, L, O, I, kw) in CASES.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **case(data_seed, L, O, I, **kw))
        print("wrote", name)


if __name__ == "__main__":
    main()
