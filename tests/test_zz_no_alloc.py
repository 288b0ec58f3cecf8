"""hot_hla_tokenwise_static: the entry point that allocates nothing (its kernels' scratch is a fixed
array inside the library's device code) must give, bit for bit, what hot_hla_tokenwise gives with a
caller-provided workspace -- on two calls in a row that share the array, the second on a smaller
input, for every statistic the scratch holds (per-tensor slots, per-channel maxima, SAWB sums)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import hot_oracle as orc

pytestmark = pytest.mark.gpu


def _both(x, n, rows, bits, rounding, scale, seed):
    from hot_amd import ops
    ref = ops.hla_tokenwise(x, n, rows, bits=bits, rounding=rounding, scale=scale, seed=seed)
    got = ops.hla_tokenwise(x, n, rows, bits=bits, rounding=rounding, scale=scale, seed=seed, static_scratch=True)
    torch.cuda.synchronize()
    return ref, got


@pytest.mark.parametrize("scale,rounding,dtype", [
    ("tensor", "nearest", torch.bfloat16),
    ("row", "stoch", torch.float32),
    ("sawb", "nearest", torch.bfloat16),
])
def test_static_scratch_matches_workspace_entry_point(gpu, scale, rounding, dtype):
    g = torch.Generator().manual_seed(17)
    n, rows = orc.hla_rows(64)
    rows = [int(v) for v in rows]
    # first call: 40 token blocks x 1096 channels (ragged last strip); second call, right behind it on
    # the same array: 6 blocks x 264 channels with values a hundred times smaller, so that a
    # statistic left over from the first call would change every step and code
    big = (torch.randn(2560, 1096, generator=g) * 3.0).to(dtype).to(gpu)
    small = (torch.randn(384, 264, generator=g) * 0.03).to(dtype).to(gpu)
    for x in (big, small):
        (codes, steps, kout), (codes_s, steps_s, kout_s) = _both(x, n, rows, 8, rounding, scale, seed=5)
        assert kout == kout_s
        assert torch.equal(steps, steps_s)
        assert torch.equal(codes, codes_s)
    # ... and against the oracle for the second (smaller) call
    mode = {"tensor": orc.SCALE_TENSOR, "row": orc.SCALE_ROW, "sawb": orc.SCALE_SAWB}[scale]
    rnd = orc.ROUND_STOCH if rounding == "stoch" else orc.ROUND_NEAREST
    tt = np.ascontiguousarray(orc.fwht_blocks_first(small.float().cpu().numpy(), n, np.asarray(rows)).T)
    q_ref, s_ref = orc.quant(tt, 8, mode, rnd, seed=5, stream=orc.STREAM_GW,
                             index=orc.colwise_rng_index(small.shape[1], small.shape[0] // n, rows))
    assert np.array_equal(codes_s.cpu().numpy()[:, :kout], q_ref)
    assert np.array_equal(steps_s.cpu().numpy(), np.atleast_1d(s_ref).astype(np.float32).reshape(-1))


def test_static_scratch_limits(gpu):
    """Sizes beyond the built-in array are refused with a clear message, before anything is launched."""
    from hot_amd import _lib, ops
    x = torch.zeros(512, 64, device=gpu)
    n, rows = orc.hla_rows(256)
    with pytest.raises(_lib.HotError, match="token blocks above 128"):
        ops.hla_tokenwise(x, 256, [int(v) for v in rows], static_scratch=True)
    wide = torch.zeros(16, _lib.HOT_STATIC_MAX_CHANNELS + 8, device=gpu)
    with pytest.raises(_lib.HotError, match="channels exceed"):
        ops.hla_tokenwise(wide, 16, list(range(16)), static_scratch=True)
    # the largest channel count it takes
    edge = torch.randn(32, _lib.HOT_STATIC_MAX_CHANNELS, device=gpu)
    a = ops.hla_tokenwise(edge, 16, list(range(8)), scale="row")
    b = ops.hla_tokenwise(edge, 16, list(range(8)), scale="row", static_scratch=True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
