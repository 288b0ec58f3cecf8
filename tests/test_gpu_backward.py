"""Parity of the fused path (hot_abc_forward + hot_linear_backward through the
C ABI, and the Python drop-in surface above it) with the CPU oracle and with
the op-for-op port of the reference's fake-quant path.

Bars: integer stages bit-exact under round-to-nearest (and, because both sides
share the counter-based generator, under stochastic rounding too); fp32 g_x /
g_W equal to the canonical oracle and within 1e-3 relative Frobenius error of
the fake-quant port."""
import numpy as np
import pytest
import torch

from oracle import fakequant_port as fq
from oracle import hot_oracle as orc

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3   # north-star tolerance on final fp32 g_x / g_W


def rel(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300)


def make_case(L, O, I, seed=0, dtype=torch.float32, outliers=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(L, I, generator=g)
    w = (torch.rand(O, I, generator=g) * 2 - 1) / I ** 0.5
    gy = torch.randn(L, O, generator=g) * 1e-3
    if outliers:
        gy = torch.where(torch.rand(L, O, generator=g) < 0.01, gy * 50, gy)
    return x.to(dtype), w.to(dtype), gy.to(dtype)


def both_configs(L, rule="python", max_block=64, **kw):
    from hot_amd import ops
    ocfg = orc.HotConfig.python_rule(L, **kw) if rule == "python" else orc.HotConfig.paper(16, 8, **kw)
    if ocfg.hla_n > max_block:
        n, rows = orc.hla_rows(64)
        ocfg.hla_n, ocfg.hla_rows = n, tuple(int(v) for v in rows)
    opt = ops.HotOptions(n_o=ocfg.n_o, hla_n=ocfg.hla_n, hla_rows=ocfg.hla_rows, gx_bits=ocfg.gx_bits,
                         w_bits=ocfg.w_bits, gw_bits=ocfg.gw_bits, act_bits=ocfg.act_bits,
                         gx_round=ocfg.gx_round, w_round=ocfg.w_round, gw_round=ocfg.gw_round,
                         act_round=ocfg.act_round, gx_scale=ocfg.gx_scale, w_scale=ocfg.w_scale,
                         gw_scale=ocfg.gw_scale, act_scale=ocfg.act_scale, seed=ocfg.seed)
    return ocfg, opt


def sum_in_ranges(parts, ranges):
    """fp32 sum of per-sample gradients in the order of the batched entry point: `ranges` ranges of
    ceil(B / ranges) consecutive samples, each from zero in sample order, then the range sums in order."""
    per = -(-len(parts) // ranges)
    sums = []
    for lo in range(0, len(parts), per):
        acc = np.zeros_like(parts[0])
        for p in parts[lo:lo + per]:
            acc = (acc + p).astype(np.float32)
        sums.append(acc)
    total = sums[0]
    for s in sums[1:]:
        total = (total + s).astype(np.float32)
    return total


def run_both(x, w, gy, ocfg, opt, gpu):
    from hot_amd import ops
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    gx, gw = ops.linear_backward(gy.to(gpu), w.to(gpu), xq, sx, opt)
    xq_ref, sx_ref = orc.abc_forward(x.float().numpy(), ocfg)
    tr = orc.linear_backward(gy.float().numpy(), w.float().numpy(), xq_ref, sx_ref, ocfg)
    lp = xq_ref.shape[0]
    got_xq = xq.cpu().numpy()
    assert np.array_equal(got_xq[:, :lp], xq_ref.T) and not got_xq[:, lp:].any()
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    return gx, gw, tr


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(448, 192, 160), (64 * 5, 208, 72), (128, 2304, 768)])
@pytest.mark.parametrize("variant", [
    dict(),                                                                       # INT4 / INT8, nearest, per tensor
    dict(gx_bits=8, w_bits=8),
    dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW),                         # per token / per channel
    dict(gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, seed=99),            # stoch_quantizer
    dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
         gw_scale=orc.SCALE_ROW, seed=7),                                         # norm_quantizer
    dict(w_scale=orc.SCALE_SAWB, act_scale=orc.SCALE_SAWB),                       # canonical W / x recipe
    dict(gw_bits=4, act_bits=4),
])
def test_backward_matches_oracle(gpu, dtype, shape, variant):
    L, O, I = shape
    x, w, gy = make_case(L, O, I, seed=L + O, dtype=dtype)
    ocfg, opt = both_configs(L, **variant)
    gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
    if dtype == torch.float32:
        # same IEEE operations in the same order on both sides
        assert np.array_equal(gx.cpu().numpy(), tr.g_x)
        assert np.array_equal(gw.cpu().numpy(), tr.g_w)
    else:
        assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dtype))
        assert torch.equal(gw.cpu(), torch.from_numpy(tr.g_w).to(dtype))


@pytest.mark.parametrize("variant", [dict(), dict(gw_scale=orc.SCALE_ROW, gx_bits=8, w_bits=8)])
def test_backward_split_k(gpu, variant):
    """Few output tiles and a long reduction (L' = 2304): the g_W GEMM cuts K into ranges that meet
    in the workspace and a second kernel adds up.  Run twice on one (dirty) workspace."""
    from hot_amd import ops
    L, O, I = 4096, 256, 256
    x, w, gy = make_case(L, O, I, seed=5)
    ocfg, opt = both_configs(L, **variant)
    assert opt.lprime(L) >= 2048
    gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
    assert np.array_equal(gx.cpu().numpy(), tr.g_x) and np.array_equal(gw.cpu().numpy(), tr.g_w)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    ws = torch.empty(1 << 26, dtype=torch.uint8, device=gpu)
    for _ in range(2):
        gx2, gw2 = ops.linear_backward(gy.to(gpu), w.to(gpu), xq, sx, opt, workspace=ws)
        assert np.array_equal(gx2.cpu().numpy(), tr.g_x) and np.array_equal(gw2.cpu().numpy(), tr.g_w)


def test_backward_paper_rule(gpu):
    L, O, I = 512, 256, 128
    x, w, gy = make_case(L, O, I, seed=1)
    ocfg, opt = both_configs(L, rule="paper")
    assert (opt.hla_n, opt.hla_r) == (16, 8)
    gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
    assert np.array_equal(gx.cpu().numpy(), tr.g_x) and np.array_equal(gw.cpu().numpy(), tr.g_w)


def test_backward_no_hla_for_odd_token_counts(gpu):
    """L = 49 (the reference harness' token count) and L = 197: n = 1, r = 1."""
    for L in (49, 197):
        x, w, gy = make_case(L, 128, 64, seed=L)
        ocfg, opt = both_configs(L)
        assert opt.hla_n == 1
        gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
        assert np.array_equal(gx.cpu().numpy(), tr.g_x) and np.array_equal(gw.cpu().numpy(), tr.g_w)


def test_backward_against_fakequant_port(gpu):
    """The reference's own evaluation order (dense matmul transforms): final
    fp32 gradients within 1e-3 relative Frobenius error."""
    L, O, I = 1344, 768, 384          # 1344 = 64 * 21: the python rule gives n = 64, r = 36
    x, w, gy = fq.config1_inputs(L, O, I, seed=0)
    ocfg, opt = both_configs(L)
    gx, gw, _ = run_both(x, w, gy, ocfg, opt, gpu)
    h_out, h_bs = fq.matrices(L, O)
    assert h_bs.shape == (len(ocfg.hla_rows), ocfg.hla_n) == (36, 64)
    xq, sx = fq.setup_context(x, h_bs, fq.PortConfig())
    gi_ref, gw_ref = fq.backward(gy, w, xq, sx, h_out, h_bs, fq.PortConfig())
    assert rel(gx.cpu().numpy(), gi_ref.numpy()) < REL_TOL
    assert rel(gw.cpu().numpy(), gw_ref.numpy()) < REL_TOL


def test_bf16_inputs_against_the_reference_bf16_evaluation(gpu):
    """With bf16 weights the reference evaluates the whole backward in bf16 (utils/quant_matmul.py:218-220:
    H cast to bf16, transform matmuls, quantiser arithmetic and the "integer" matmuls in bf16, whose
    results are rounded to 8 significant bits); the native path widens the same bf16 inputs to fp32,
    transforms and quantises in fp32 and accumulates in int32.  The two therefore differ by the
    reference's own bf16 rounding noise.  Pinned here at the ViT-B fc1 size:
      * native (fp32 out) is within 1e-3 of the reference's evaluation order run in fp32 on the same
        bf16 inputs;
      * the distance native <-> reference-in-bf16 is no larger than the distance of the reference's
        bf16 evaluation from its own fp32 evaluation (it IS that noise), and stays below 10 %."""
    from hot_amd import ops
    L, O, I = 12608, 3072, 768
    x, w, gy = fq.config1_inputs(L, O, I, seed=0)
    xb, wb, gb = x.to(torch.bfloat16), w.to(torch.bfloat16), gy.to(torch.bfloat16)
    ocfg, opt = both_configs(L)
    xq, sx = ops.abc_forward(xb.to(gpu), opt)
    gx, gw = ops.linear_backward(gb.to(gpu), wb.to(gpu), xq, sx, opt, out_dtype=torch.float32)
    gx, gw = gx.cpu().numpy(), gw.cpu().numpy()
    out = {}
    for dt in (torch.float32, torch.bfloat16):
        h_out, h_bs = fq.matrices(L, O, dt)
        xq_r, sx_r = fq.setup_context(xb.to(dt), h_bs, fq.PortConfig())
        gi, gwr = fq.backward(gb.to(dt), wb.to(dt), xq_r, sx_r, h_out, h_bs, fq.PortConfig())
        assert gi.dtype == dt and gwr.dtype == dt
        out[dt] = (gi.float().numpy(), gwr.float().numpy())
    d32 = (rel(gx, out[torch.float32][0]), rel(gw, out[torch.float32][1]))
    d16 = (rel(gx, out[torch.bfloat16][0]), rel(gw, out[torch.bfloat16][1]))
    own = (rel(out[torch.bfloat16][0], out[torch.float32][0]), rel(out[torch.bfloat16][1], out[torch.float32][1]))
    print("native vs reference order in fp32: g_x %.2e g_W %.2e; vs its bf16 evaluation: g_x %.2e g_W %.2e; "
          "reference bf16 vs fp32: g_x %.2e g_W %.2e" % (d32 + d16 + own))
    assert d32[0] < REL_TOL and d32[1] < REL_TOL
    assert d16[0] <= own[0] * 1.05 + 1e-3 and d16[1] <= own[1] * 1.05 + 1e-3
    assert d16[0] < 0.1 and d16[1] < 0.1


def test_vit_fc1_full_size(gpu):
    """The headline workload (ViT-B fc1) at full size (L = 12608, O = 3072, I = 768):
    bit-exact against the canonical oracle, 1e-3 against the fake-quant port."""
    L, O, I = 12608, 3072, 768
    x, w, gy = fq.config1_inputs(L, O, I, seed=0)
    ocfg, opt = both_configs(L)
    assert (opt.hla_n, opt.hla_r) == (64, 36)
    gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
    assert np.array_equal(gx.cpu().numpy(), tr.g_x)
    assert np.array_equal(gw.cpu().numpy(), tr.g_w)
    h_out, h_bs = fq.matrices(L, O)
    xq, sx = fq.setup_context(x, h_bs, fq.PortConfig())
    gi_ref, gw_ref = fq.backward(gy, w, xq, sx, h_out, h_bs, fq.PortConfig())
    assert rel(gx.cpu().numpy(), gi_ref.numpy()) < REL_TOL
    assert rel(gw.cpu().numpy(), gw_ref.numpy()) < REL_TOL
    # the entry point that also returns the bias gradient: same gradients; on integer-valued g_y the
    # column sums are exact whatever the order of the additions
    from hot_amd import ops
    xq_d, sx_d = ops.abc_forward(x.to(gpu), opt)
    gx_b, gw_b, gb = ops.linear_backward(gy.to(gpu), w.to(gpu), xq_d, sx_d, opt, bias_grad=True)
    assert torch.equal(gx_b, gx) and torch.equal(gw_b, gw)
    ref = gy.double().sum(dim=0)
    assert float((gb.double().cpu() - ref).abs().max()) <= L * 2.0 ** -24 * float(gy.double().abs().sum(dim=0).max())
    gi = torch.randint(-8, 9, (L, O), generator=torch.Generator().manual_seed(5)).float()
    _, _, gbi = ops.linear_backward(gi.to(gpu), w.to(gpu), xq_d, sx_d, opt, bias_grad=True)
    assert torch.equal(gbi.cpu(), gi.sum(dim=0))


@pytest.mark.parametrize("shape", [(8192, 11008, 4096), (8192, 4096, 11008)])
def test_llama_shapes_properties(gpu, shape):
    """Llama-7B MLP shapes, bf16, too large for the CPU oracle: checked through
    size-independent properties.
      * scaling g_y by a power of two scales both gradients by exactly that
        factor (absmax quantisation commutes with it);
      * INT8 everywhere with all coefficients kept approximates the bf16 matmul."""
    from hot_amd import ops
    L, O, I = shape
    g = torch.Generator(device="cpu").manual_seed(1)
    # unit-variance g_y keeps every step size far above the 1e-11 guard added to it,
    # which is the only term that does not scale
    gy = torch.randn(L, O, generator=g).to(torch.bfloat16).to(gpu)
    w = ((torch.rand(O, I, generator=g) * 2 - 1) / I ** 0.5).to(torch.bfloat16).to(gpu)
    x = torch.randn(L, I, generator=g).to(torch.bfloat16).to(gpu)
    _, opt = both_configs(L, rule="paper")
    xq, sx = ops.abc_forward(x, opt)
    gx, gw = ops.linear_backward(gy, w, xq, sx, opt, out_dtype=torch.float32)
    gx4, gw4 = ops.linear_backward(gy * 4, w, xq, sx, opt, out_dtype=torch.float32)
    assert torch.equal(gx4, gx * 4) and torch.equal(gw4, gw * 4)
    full = ops.HotOptions(hla_n=16, hla_rows=tuple(range(16)), gx_bits=8, w_bits=8, gw_bits=8, act_bits=8)
    xq8, sx8 = ops.abc_forward(x, full)
    gx8, gw8 = ops.linear_backward(gy, w, xq8, sx8, full, out_dtype=torch.float32)
    ref_gx = gy.float() @ w.float()
    ref_gw = gy.float().T @ x.float()
    assert float((gx8 - ref_gx).norm() / ref_gx.norm()) < 0.03
    assert float((gw8 - ref_gw).norm() / ref_gw.norm()) < 0.03


def test_hlq_backward_op_surface(gpu):
    """HLQ_backward.backward(Go, W, X, 0, 0, 16, per_token) -> (gx, gw, 4 floats)."""
    from hot_amd import HLQ_backward
    L, O, I = 192, 3072, 768
    rng = np.random.default_rng(2023)
    X = torch.tensor(rng.lognormal(1.0, 0.1, (L, I)), dtype=torch.float32)
    Go = torch.tensor(rng.lognormal(1.0, 0.1, (L, O)), dtype=torch.float32)
    W = torch.tensor(rng.lognormal(1.0, 0.1, (O, I)), dtype=torch.float32)
    for per_token in (True, False):
        gx, gw, times = HLQ_backward.backward(Go.to(gpu), W.to(gpu), X.to(gpu), 0, 0, 16, per_token)
        assert gx.shape == (L, I) and gw.shape == (O, I) and gx.dtype == Go.dtype
        # [transform-only passes, transform + quantise passes, both GEMMs, 0: dequantisation is fused]
        assert isinstance(times, list) and len(times) == 4 and all(isinstance(t, float) for t in times)
        assert all(t > 0 for t in times[:3]) and times[3] == 0.0
        opt = HLQ_backward.options(L, 16, per_token)
        ocfg = orc.HotConfig(n_o=16, hla_n=opt.hla_n, hla_rows=opt.hla_rows, gx_round=orc.ROUND_STOCH,
                             gx_scale=orc.SCALE_ROW if per_token else orc.SCALE_TENSOR, seed=HLQ_backward.seed)
        xq_ref, sx_ref = orc.abc_forward(X.numpy(), ocfg)
        tr = orc.linear_backward(Go.numpy(), W.numpy(), xq_ref, sx_ref, ocfg)
        assert np.array_equal(gx.cpu().numpy(), tr.g_x) and np.array_equal(gw.cpu().numpy(), tr.g_w)
    with pytest.raises(RuntimeError, match="Go must be contiguous!"):
        HLQ_backward.backward(Go.to(gpu).t().contiguous().t(), W.to(gpu), X.to(gpu), 0, 0, 16, True)
    with pytest.raises(RuntimeError, match="X must be 2D!"):
        HLQ_backward.backward(Go.to(gpu), W.to(gpu), X.to(gpu)[None], 0, 0, 16, True)


@pytest.fixture
def fresh_args():
    from hot_amd import args
    saved = {k: getattr(args, k) for k in dir(args) if not k.startswith("_")}
    args.hot_recipe()          # the module defaults describe a plain layer, as the reference's do
    yield args
    for k, v in saved.items():
        setattr(args, k, v)


def test_hq_linear_training_step(gpu, fresh_args):
    """HQ_Linear forward (full precision) + backward (HOT) through autograd."""
    from hot_amd.quant_matmul import HQ_Linear
    L, I, O = 256, 96, 128
    fresh_args.hla_max_block = 64          # 256 tokens: blocks of 64 (one-pass kernels); the default is below
    torch.manual_seed(0)
    lin = HQ_Linear(I, O).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    y = lin(x)
    assert torch.allclose(y, torch.nn.functional.linear(x, lin.weight, lin.bias))
    gy = torch.randn(L, O, device=gpu) * 1e-3
    y.backward(gy)
    ocfg, _ = both_configs(L)
    xq_ref, sx_ref = orc.abc_forward(x.detach().cpu().numpy(), ocfg)
    tr = orc.linear_backward(gy.cpu().numpy(), lin.weight.detach().cpu().numpy(), xq_ref, sx_ref, ocfg)
    assert np.array_equal(x.grad.cpu().numpy(), tr.g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), tr.g_w)
    assert torch.allclose(lin.bias.grad, gy.sum(0), rtol=1e-5, atol=1e-8)
    assert lin.hadamard_bs.shape == (36, 64)
    # default: the reference's rule without a cap, 256 tokens -> one block of 256, 136 rows kept
    fresh_args.hla_max_block = 8192
    lin.zero_grad()
    x2 = x.detach().clone().requires_grad_(True)
    lin(x2).backward(gy)
    ocfg = orc.HotConfig.python_rule(L)
    assert (ocfg.hla_n, len(ocfg.hla_rows)) == (256, 136)
    xq_ref, sx_ref = orc.abc_forward(x2.detach().cpu().numpy(), ocfg)
    tr = orc.linear_backward(gy.cpu().numpy(), lin.weight.detach().cpu().numpy(), xq_ref, sx_ref, ocfg)
    assert np.array_equal(x2.grad.cpu().numpy(), tr.g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), tr.g_w)
    assert lin.hadamard_bs.shape == (1, 1)          # placeholder beyond 64 tokens per block


@pytest.mark.parametrize("mode", ["per_sample", "flatten"])
def test_hq_linear_3d_input(gpu, fresh_args, mode):
    """[B, L, C] activations: per-sample steps as in the reference (vmap over
    the batch, utils/quant_matmul.py:118-122) or flattened tokens."""
    from hot_amd.quant_matmul import HQ_Linear
    fresh_args.batched_mode = mode
    B, L, I, O = 3, 64, 48, 80
    torch.manual_seed(1)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(B, L, I, device=gpu, requires_grad=True)
    gy = torch.randn(B, L, O, device=gpu) * 1e-3
    lin(x).backward(gy)
    wn = lin.weight.detach().cpu().numpy()
    if mode == "per_sample":
        from hot_amd import ops
        ocfg, opt = both_configs(L)
        gxs, gws = [], []
        for b in range(B):
            xq_ref, sx_ref = orc.abc_forward(x[b].detach().cpu().numpy(), ocfg)
            tr = orc.linear_backward(gy[b].cpu().numpy(), wn, xq_ref, sx_ref, ocfg)
            gxs.append(tr.g_x)
            gws.append(tr.g_w)
        assert np.array_equal(x.grad.cpu().numpy(), np.stack(gxs))
        # fp32 sum over the samples, in the order the library states
        assert np.array_equal(lin.weight.grad.cpu().numpy(), sum_in_ranges(gws, ops.backward_batched_ranges(B, L, O, I, opt)))
    else:
        ocfg, _ = both_configs(B * L)
        xq_ref, sx_ref = orc.abc_forward(x.detach().reshape(B * L, I).cpu().numpy(), ocfg)
        tr = orc.linear_backward(gy.reshape(B * L, O).cpu().numpy(), wn, xq_ref, sx_ref, ocfg)
        assert np.array_equal(x.grad.cpu().numpy().reshape(B * L, I), tr.g_x)
        assert np.array_equal(lin.weight.grad.cpu().numpy(), tr.g_w)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,O,I,variant", [
    (5, 197, 208, 72, dict()),                                                    # ViT tokens: no block divides 197
    (3, 64, 192, 160, dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW)),      # n = 64, r = 36 inside every sample
    (4, 196, 96, 264, dict(gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, act_round=orc.ROUND_STOCH, seed=21)),
    (2, 200, 128, 96, dict(w_scale=orc.SCALE_SAWB, act_scale=orc.SCALE_SAWB)),
    (7, 48, 64, 40, dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
                         gw_scale=orc.SCALE_ROW, gx_bits=8, w_bits=8, seed=5)),
    (130, 197, 128, 64, dict()),                                                  # more samples than a ViT batch
    (6, 197, 80, 136, dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
                           act_round=orc.ROUND_STOCH, seed=9)),                      # one-token blocks, stochastic
    (1, 128, 48, 24, dict()),                                                     # a batch of one
    (3, 64, 16, 8, dict(gw_scale=orc.SCALE_ROW)),                                 # one block per sample, smallest widths
    (2, 576, 256, 384, dict(gx_bits=8, w_bits=8)),                                # 324 codes per sample: three stages per group
])
def test_backward_batched_matches_oracle(gpu, dtype, B, T, O, I, variant):
    """3-D activations through the batched entry points (one call per layer, one set of steps per
    sample): activation buffer, g_x and the summed g_W equal the per-sample oracle bit for bit."""
    from hot_amd import ops
    g = torch.Generator().manual_seed(B * T + O)
    mag = 10.0 ** (torch.rand(B, 1, 1, generator=g) * 3 - 3)                       # samples of very different size
    x = (torch.randn(B, T, I, generator=g) * (mag * 100)).to(dtype)
    w = ((torch.rand(O, I, generator=g) * 2 - 1) / I ** 0.5).to(dtype)
    gy = (torch.randn(B, T, O, generator=g) * mag).to(dtype)
    ocfg = orc.HotConfig.python_rule(T, **variant)
    opt = ops.HotOptions(n_o=ocfg.n_o, hla_n=ocfg.hla_n, hla_rows=ocfg.hla_rows, gx_bits=ocfg.gx_bits, w_bits=ocfg.w_bits,
                         gw_bits=ocfg.gw_bits, act_bits=ocfg.act_bits, gx_round=ocfg.gx_round, w_round=ocfg.w_round,
                         gw_round=ocfg.gw_round, act_round=ocfg.act_round, gx_scale=ocfg.gx_scale, w_scale=ocfg.w_scale,
                         gw_scale=ocfg.gw_scale, act_scale=ocfg.act_scale, seed=ocfg.seed)
    xq, sx = ops.abc_forward_batched(x.to(gpu), opt)
    gx, gw = ops.linear_backward_batched(gy.to(gpu), w.to(gpu), xq, sx, opt)
    xq_ref, sx_ref = orc.abc_forward_batched(x.float().numpy(), ocfg)
    ranges = ops.backward_batched_ranges(B, T, O, I, opt)
    assert 1 <= ranges <= B
    gx_ref, gw_ref, _ = orc.linear_backward_batched(gy.float().numpy(), w.float().numpy(), xq_ref, sx_ref, ocfg, gw_ranges=ranges)
    kg = ops.kpad_group(T, opt)
    tp = xq_ref.shape[1]
    got = xq.cpu().numpy().reshape(I, B, kg)
    assert kg % 128 == 0 and kg >= tp
    assert np.array_equal(got[:, :, :tp], xq_ref.transpose(2, 0, 1)) and not got[:, :, tp:].any()
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    assert torch.equal(gx.cpu(), torch.from_numpy(gx_ref).to(dtype))
    assert torch.equal(gw.cpu(), torch.from_numpy(gw_ref).to(dtype))


def test_hq_conv2d_matches_oracle(gpu, fresh_args):
    """HQ_Conv2d = im2col + the linear path per sample (utils/quant_matmul.py:426-488): the weight
    gradient is the sum of the per-sample oracle results, the input gradient their fold."""
    from hot_amd.quant_matmul import HQ_Conv2d
    B, C, H, W, O, k = 2, 8, 16, 16, 32, 2
    torch.manual_seed(2)
    conv = HQ_Conv2d(C, O, kernel_size=k, stride=k).to(gpu)
    ref = torch.nn.Conv2d(C, O, kernel_size=k, stride=k).to(gpu)
    ref.load_state_dict({n: p for n, p in conv.state_dict().items() if n in ("weight", "bias")})
    x = torch.randn(B, C, H, W, device=gpu, requires_grad=True)
    y = conv(x)
    assert torch.allclose(y, ref(x), atol=1e-5, rtol=1e-5)
    G = torch.randn_like(y) * 1e-3
    y.backward(G)
    L = (H // k) * (W // k)
    ocfg, _ = both_configs(L)
    cols = torch.nn.functional.unfold(x.detach().cpu(), k, stride=k).transpose(1, 2)       # [B, L, C k k]
    gy = G.cpu().flatten(2).transpose(1, 2)                                                # [B, L, O]
    wn = conv.weight.detach().cpu().reshape(O, -1).numpy()
    gw, gcols = 0, []
    for b in range(B):
        xq_ref, sx_ref = orc.abc_forward(cols[b].contiguous().numpy(), ocfg)
        tr = orc.linear_backward(gy[b].contiguous().numpy(), wn, xq_ref, sx_ref, ocfg)
        gw = gw + tr.g_w
        gcols.append(torch.from_numpy(tr.g_x))
    # stride == kernel: the patches do not overlap, so the fold only moves values
    gx = torch.nn.functional.fold(torch.stack(gcols).transpose(1, 2), (H, W), k, stride=k)
    assert np.array_equal(x.grad.cpu().numpy(), gx.numpy())
    assert rel(conv.weight.grad.cpu().reshape(O, -1).numpy(), gw) < 1e-6
    assert torch.allclose(conv.bias.grad.cpu(), G.cpu().sum((0, 2, 3)), rtol=1e-4, atol=1e-7)


def test_hq_conv2d_overlapping_patches(gpu, fresh_args):
    """Kernel 3, stride 1, padding 1: the unfold path (the non-overlapping case above is a plain
    permutation); the input gradient is the fold (a sum over overlapping patches) of the oracle's."""
    from hot_amd.quant_matmul import HQ_Conv2d
    B, C, H, W, O, k = 2, 8, 8, 8, 16, 3
    torch.manual_seed(4)
    conv = HQ_Conv2d(C, O, kernel_size=k, stride=1, padding=1).to(gpu)
    x = torch.randn(B, C, H, W, device=gpu, requires_grad=True)
    y = conv(x)
    assert torch.allclose(y, torch.nn.functional.conv2d(x, conv.weight, conv.bias, padding=1), atol=1e-5, rtol=1e-5)
    G = torch.randn_like(y) * 1e-3
    y.backward(G)
    L = H * W
    ocfg, _ = both_configs(L)
    cols = torch.nn.functional.unfold(x.detach().cpu(), k, padding=1).transpose(1, 2)      # [B, L, C k k]
    gy = G.cpu().flatten(2).transpose(1, 2)
    wn = conv.weight.detach().cpu().reshape(O, -1).numpy()
    gw, gcols = 0, []
    for b in range(B):
        xq_ref, sx_ref = orc.abc_forward(cols[b].contiguous().numpy(), ocfg)
        tr = orc.linear_backward(gy[b].contiguous().numpy(), wn, xq_ref, sx_ref, ocfg)
        gw = gw + tr.g_w
        gcols.append(torch.from_numpy(tr.g_x))
    gx = torch.nn.functional.fold(torch.stack(gcols).transpose(1, 2), (H, W), k, padding=1)
    assert rel(x.grad.cpu().numpy(), gx.numpy()) < 1e-6
    assert rel(conv.weight.grad.cpu().reshape(O, -1).numpy(), gw) < 1e-6



def test_lqs_then_hot_training_step(gpu, fresh_args):
    """Calibrate in the plain setting, then take a HOT step with the selected quantisers."""
    from hot_amd import lqs, utils as hutils
    from hot_amd.quant_matmul import HQ_Linear
    torch.manual_seed(3)
    model = torch.nn.Sequential(torch.nn.Linear(64, 128), torch.nn.GELU(), torch.nn.Linear(128, 32)).to(gpu)
    hutils.replace_layers(model, torch.nn.Linear, HQ_Linear)
    hutils.name_layers(model)
    fresh_args.layer_quant_dict.clear()
    batches = [(torch.randn(256, 64, device=gpu), torch.randint(0, 32, (256,), device=gpu))]
    chosen = lqs.calibrate(model, batches, torch.nn.CrossEntropyLoss())
    assert set(chosen) == {"0_gx", "0_gw", "2_gx", "2_gw"}
    fresh_args.quantAuto = True
    model.zero_grad()
    x, t = batches[0]
    torch.nn.functional.cross_entropy(model(x), t).backward()
    hot = [p.grad.clone() for p in model.parameters()]
    # the same step in the plain setting: the HOT gradients approximate it
    for k_ in ("TransformGogi", "TransformWgt", "TransformGogw", "TransformInput"):
        setattr(fresh_args, k_, False)
    for k_ in ("quantBWDGogi", "quantBWDWgt", "quantBWDGogw", "quantBWDAct"):
        setattr(fresh_args, k_, "no")
    model.zero_grad()
    torch.nn.functional.cross_entropy(model(x), t).backward()
    for h, p in zip(hot, model.parameters()):
        cos = torch.nn.functional.cosine_similarity(h.flatten(), p.grad.flatten(), dim=0)
        # random tokens have no low-sequency structure: keeping about half the rows keeps about half the
        # energy of g_W, a cosine near 0.7
        assert float(cos) > 0.55, float(cos)


def test_backward_errors(gpu):
    from hot_amd import ops
    from hot_amd._lib import HotError
    x, w, gy = make_case(128, 64, 32)
    _, opt = both_configs(128)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    with pytest.raises(RuntimeError):
        ops.linear_backward(gy.to(gpu), w.to(gpu)[:32].contiguous(), xq, sx, opt)        # O mismatch
    bad = ops.HotOptions(hla_n=opt.hla_n, hla_rows=opt.hla_rows, gx_bits=4, w_bits=8)
    with pytest.raises(HotError, match="must match"):
        ops.linear_backward(gy.to(gpu), w.to(gpu), xq, sx, bad)
    with pytest.raises(HotError):
        ops.abc_forward(x.to(gpu)[:100].contiguous(), opt)                               # L % n


def test_backward_launch_orders_agree(gpu):
    """hot_backward_streams: short calls run on the caller's stream, long ones fork the library's side
    stream; cfg.streams overrides the rule; both orders give the same bits, bias gradient included."""
    from dataclasses import replace
    from hot_amd import ops
    L, O, I = 1344, 384, 192
    x, w, gy = make_case(L, O, I, seed=12, dtype=torch.bfloat16)
    _, opt = both_configs(L)
    assert ops.backward_streams(L, O, I, opt) == 1                                   # 0.3 GOP
    assert ops.backward_streams(12608, 768, 768, opt) == 1 and ops.backward_streams(12608, 2304, 768, opt) == 2
    assert ops.backward_streams(L, O, I, replace(opt, streams=2)) == 2
    assert ops.backward_streams(12608, 3072, 768, replace(opt, streams=1)) == 1
    with pytest.raises(ops.HotError, match="streams"):
        ops.linear_backward(gy.to(gpu), w.to(gpu), *ops.abc_forward(x.to(gpu), opt), replace(opt, streams=3))
    x, w, gy = x.to(gpu), w.to(gpu), gy.to(gpu)
    xq, sx = ops.abc_forward(x, opt)
    for variant in (dict(), dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH, seed=5)):
        one = ops.linear_backward(gy, w, xq, sx, replace(opt, streams=1, **variant), bias_grad=True)
        two = ops.linear_backward(gy, w, xq, sx, replace(opt, streams=2, **variant), bias_grad=True)
        for a, b in zip(one, two):
            assert torch.equal(a, b)


@pytest.mark.parametrize("streams", [1, 2])
def test_backward_in_hip_graph(gpu, streams):
    """The whole call -- on the caller's stream alone, or with the library's side stream forked and
    joined by events -- is capturable; every replay, with eager work in between, equals the eager result."""
    from dataclasses import replace
    from hot_amd import ops
    L, O, I = 1344, 384, 192
    x, w, gy = make_case(L, O, I, seed=11, dtype=torch.bfloat16)
    _, opt = both_configs(L)
    opt = replace(opt, streams=streams)
    x, w, gy = x.to(gpu), w.to(gpu), gy.to(gpu)
    xq, sx = ops.abc_forward(x, opt)
    ws = torch.empty(1 << 26, dtype=torch.uint8, device=gpu)
    eager = ops.linear_backward(gy, w, xq, sx, opt, workspace=ws)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up on a side stream, as capture requires
        ops.linear_backward(gy, w, xq, sx, opt, workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ops.linear_backward(gy, w, xq, sx, opt, workspace=ws)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out[0], eager[0]) and torch.equal(out[1], eager[1])
        again = ops.linear_backward(gy, w, xq, sx, opt, workspace=ws)      # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(again[0], eager[0]) and torch.equal(again[1], eager[1])


def test_backward_large_block_in_hip_graph(gpu):
    """Token blocks of 1024 (the make_WHT rule on 2048 tokens) take the two-level path, whose row table
    is written by kernels that carry the rows in their arguments: the call records into a HIP graph like
    any other, replays equal the eager result and the oracle, also after the host arrays that held the
    rows during capture are gone and the workspace has been scribbled over."""
    from hot_amd import ops
    L, O, I = 2048, 128, 64
    x, w, gy = make_case(L, O, I, seed=13, dtype=torch.float32)
    ocfg = orc.HotConfig.python_rule(L)
    assert ocfg.hla_n == 2048 and len(ocfg.hla_rows) == 528
    n, rows = orc.hla_rows(1024)
    ocfg.hla_n, ocfg.hla_rows = n, tuple(int(v) for v in rows)
    opt = ops.HotOptions(n_o=16, hla_n=n, hla_rows=ocfg.hla_rows)
    xd, wd, gyd = x.to(gpu), w.to(gpu), gy.to(gpu)
    xq, sx = ops.abc_forward(xd, opt)
    xq_ref, sx_ref = orc.abc_forward(x.numpy(), ocfg)
    tr = orc.linear_backward(gy.numpy(), w.numpy(), xq_ref, sx_ref, ocfg)
    need = 1 << 26
    ws = torch.empty(need, dtype=torch.uint8, device=gpu)
    eager = ops.linear_backward(gyd, wd, xq, sx, opt, workspace=ws)
    torch.cuda.synchronize()
    assert np.array_equal(eager[0].cpu().numpy(), tr.g_x) and np.array_equal(eager[1].cpu().numpy(), tr.g_w)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.linear_backward(gyd, wd, xq, sx, opt, workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    opt_cap = ops.HotOptions(n_o=16, hla_n=n, hla_rows=ocfg.hla_rows)       # its own C arrays, dropped below
    with torch.cuda.graph(graph):
        out = ops.linear_backward(gyd, wd, xq, sx, opt_cap, workspace=ws)
    del opt_cap
    import gc
    gc.collect()
    for _ in range(3):
        ws.fill_(0x5A)                                   # the row table in the workspace is rebuilt by the replay
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out[0].cpu().numpy(), tr.g_x) and np.array_equal(out[1].cpu().numpy(), tr.g_w)
        again = ops.linear_backward(gyd, wd, xq, sx, opt, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(again[0], eager[0]) and torch.equal(again[1], eager[1])


def test_small_vit_with_hot_layers(gpu, fresh_args):
    """A whole (small) ViT with every Linear / Conv2d swapped: LQS calibration, then one HOT step whose
    parameter gradients point the same way as the full-precision ones."""
    from hot_amd import lqs, utils as hutils
    from hot_amd.quant_matmul import HQ_Conv2d, HQ_Linear
    from hot_amd.vit import ViT
    torch.manual_seed(5)
    model = ViT(image=32, patch=8, dim=64, depth=2, heads=4, mlp=128, classes=10, channels=8).to(gpu)
    hutils.replace_layers(model, torch.nn.Conv2d, HQ_Conv2d)
    hutils.replace_layers(model, torch.nn.Linear, HQ_Linear)
    hutils.name_layers(model)
    n_hot = sum(isinstance(m, (HQ_Linear, HQ_Conv2d)) for m in model.modules())
    assert n_hot == 1 + 2 * 4 + 1
    fresh_args.batched_mode = "flatten"
    fresh_args.layer_quant_dict.clear()
    x = torch.randn(16, 8, 32, 32, device=gpu)
    t = torch.randint(0, 10, (16,), device=gpu)
    lqs.calibrate(model, [(x, t)], torch.nn.CrossEntropyLoss())
    assert len(fresh_args.layer_quant_dict) == 2 * n_hot
    fresh_args.quantAuto = True
    fresh_args.GogiQuantBit = fresh_args.weightQuantBit = 8          # a small model: keep the noise low
    model.zero_grad()
    torch.nn.functional.cross_entropy(model(x), t).backward()
    hot = {n: p.grad.clone() for n, p in model.named_parameters()}
    assert all(torch.isfinite(g).all() for g in hot.values())
    for k_ in ("TransformGogi", "TransformWgt", "TransformGogw", "TransformInput"):
        setattr(fresh_args, k_, False)
    for k_ in ("quantBWDGogi", "quantBWDWgt", "quantBWDGogw", "quantBWDAct"):
        setattr(fresh_args, k_, "no")
    model.zero_grad()
    torch.nn.functional.cross_entropy(model(x), t).backward()
    for n, p in model.named_parameters():
        if p.grad.numel() < 64:
            continue
        cos = torch.nn.functional.cosine_similarity(hot[n].flatten(), p.grad.flatten(), dim=0)
        assert float(cos) > 0.5, (n, float(cos))


@pytest.mark.parametrize("O,I", [(100, 96), (104, 100), (10, 36)])
def test_hq_linear_odd_feature_counts(gpu, fresh_args, O, I):
    """Heads and other layers whose widths are not multiples of 16: the Hadamard block along the
    out-features follows the reference's rule (largest power of two dividing them, at most 16:
    4 for 100 classes, 2 for 10) and widths that are not multiples of 8 are zero-padded on the way in."""
    from hot_amd.quant_matmul import HQ_Linear
    from hot_amd.hadamard_matmul import biggest_power2_factor_max16
    L = 192
    torch.manual_seed(7)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    lin(x).backward(gy)
    ocfg, _ = both_configs(L)
    ocfg.n_o = biggest_power2_factor_max16(O)
    assert ocfg.n_o == {100: 4, 104: 8, 10: 2}[O]
    xq_ref, sx_ref = orc.abc_forward(x.detach().cpu().numpy(), ocfg)
    tr = orc.linear_backward(gy.cpu().numpy(), lin.weight.detach().cpu().numpy(), xq_ref, sx_ref, ocfg)
    assert np.array_equal(x.grad.cpu().numpy(), tr.g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), tr.g_w)


@pytest.mark.parametrize("name", ["nearest_int4_L320_O64_I48", "stoch_row_int8_L192_O32_I40"])
def test_backward_matches_golden_fixture(gpu, name):
    """The committed fixtures (inputs, saved buffer, outputs) against the native path."""
    import os
    from hot_amd import ops
    f = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name + ".npz"))
    stoch = name.startswith("stoch")
    opt = ops.HotOptions(hla_n=int(f["hla_n"]), hla_rows=tuple(int(v) for v in f["hla_rows"]),
                         gx_bits=8 if stoch else 4, w_bits=8 if stoch else 4,
                         gx_round="stoch" if stoch else "nearest", gw_round="stoch" if stoch else "nearest",
                         gx_scale="row" if stoch else "tensor", gw_scale="row" if stoch else "tensor",
                         seed=1234 if stoch else 0)
    x, w, gy = (torch.from_numpy(f[k]).to(gpu) for k in ("x", "w", "gy"))
    xq, sx = ops.abc_forward(x, opt)
    lp = f["xq"].shape[0]
    assert np.array_equal(xq.cpu().numpy()[:, :lp], f["xq"].T) and np.array_equal(sx.cpu().numpy(), f["sx"])
    gx, gw = ops.linear_backward(gy, w, xq, sx, opt)
    assert np.array_equal(gx.cpu().numpy(), f["g_x"]) and np.array_equal(gw.cpu().numpy(), f["g_w"])


@pytest.mark.parametrize("L,O,I,variant", [
    (256, 64, 48, dict()),                                                      # n = 256, r = 136
    (384, 32, 40, dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW)),        # 384 = 128 * 3 -> n = 128
    (2048, 48, 32, dict(gw_round=orc.ROUND_STOCH, gx_round=orc.ROUND_STOCH, seed=9)),
    (8192, 32, 16, dict(w_scale=orc.SCALE_SAWB, act_scale=orc.SCALE_SAWB)),     # the Llama token count: n = 8192, r = 2080
])
def test_backward_exact_python_rule_on_large_blocks(gpu, L, O, I, variant):
    """The make_WHT rule without a cap on the block: token counts with many factors of two."""
    from hot_amd import ops
    ocfg = orc.HotConfig.python_rule(L, **variant)
    assert ocfg.hla_n == (L & -L) and ocfg.hla_n > 64
    opt = ops.HotOptions(n_o=ocfg.n_o, hla_n=ocfg.hla_n, hla_rows=ocfg.hla_rows, gx_bits=ocfg.gx_bits,
                         w_bits=ocfg.w_bits, gw_bits=ocfg.gw_bits, act_bits=ocfg.act_bits,
                         gx_round=ocfg.gx_round, w_round=ocfg.w_round, gw_round=ocfg.gw_round,
                         act_round=ocfg.act_round, gx_scale=ocfg.gx_scale, w_scale=ocfg.w_scale,
                         gw_scale=ocfg.gw_scale, act_scale=ocfg.act_scale, seed=ocfg.seed)
    x, w, gy = make_case(L, O, I, seed=L)
    gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
    assert np.array_equal(gx.cpu().numpy(), tr.g_x)
    assert np.array_equal(gw.cpu().numpy(), tr.g_w)


def _options_like(ocfg):
    from hot_amd import ops
    return ops.HotOptions(n_o=ocfg.n_o, hla_n=ocfg.hla_n, hla_rows=ocfg.hla_rows, gx_bits=ocfg.gx_bits,
                          w_bits=ocfg.w_bits, gw_bits=ocfg.gw_bits, act_bits=ocfg.act_bits,
                          gx_round=ocfg.gx_round, w_round=ocfg.w_round, gw_round=ocfg.gw_round,
                          act_round=ocfg.act_round, gx_scale=ocfg.gx_scale, w_scale=ocfg.w_scale,
                          gw_scale=ocfg.gw_scale, act_scale=ocfg.act_scale, seed=ocfg.seed)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("L,O,I,rule,variant", [
    (448, 192, 160, "python", dict()),                                             # n = 64, fused row statistic
    (64 * 5, 208, 72, "python", dict()),                                           # O short of a workgroup's 256 channels
    (64 * 37, 528, 64, "python", dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW,
                                      gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, seed=5)),   # several strips
    (448, 192, 160, "paper", dict()),                                              # n = 16, r = 8
    (197, 96, 64, "python", dict()),                                               # n = 1
    (384, 64, 40, "python", dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW)),  # n = 128
    (1024, 80, 48, "python", dict()),                                              # n = 1024: two-level path
])
def test_backward_with_bias_gradient(gpu, dtype, L, O, I, rule, variant):
    """hot_linear_backward_bias: g_x and g_W are those of hot_linear_backward bit for bit, and g_b is
    the sum of g_y over the tokens.  The reference has no code for it (autograd reduces g_y for the bias
    added at utils/quant_matmul.py:419-420), so it is pinned by the mathematics: on integer-valued g_y
    every fp32 partial sum is exact whatever the order and g_b must EQUAL the integer sum; on random
    g_y it must lie within the fp32 accumulation bound (tokens * 2^-24 * sum |g_y|) of the float64 sum,
    plus one rounding of the output type (2^-9 relative for bf16)."""
    from hot_amd import ops
    ocfg = orc.HotConfig.python_rule(L, **variant) if rule == "python" else orc.HotConfig.paper(16, 8, **variant)
    opt = _options_like(ocfg)
    x, w, gy = make_case(L, O, I, seed=3, dtype=dtype)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    gyd, wd = gy.to(gpu), w.to(gpu)
    gx0, gw0 = ops.linear_backward(gyd, wd, xq, sx, opt)
    gx1, gw1, gb = ops.linear_backward(gyd, wd, xq, sx, opt, bias_grad=True)
    assert torch.equal(gx0, gx1) and torch.equal(gw0, gw1)
    assert gb.shape == (O,) and gb.dtype == dtype
    ref = gy.double().sum(dim=0).numpy()
    bound = L * 2.0 ** -24 * gy.double().abs().sum(dim=0).numpy()
    if dtype == torch.bfloat16:
        bound = bound + 2.0 ** -8 * np.abs(ref)
    assert np.all(np.abs(gb.double().cpu().numpy() - ref) <= bound + 1e-30)
    # integer-valued g_y: exact sums (|sum| < 2^24), any dropped, doubled or misplaced block shows
    g = torch.Generator().manual_seed(11)
    gi = torch.randint(-8, 9, (L, O), generator=g).to(dtype)
    _, _, gbi = ops.linear_backward(gi.to(gpu), wd, xq, sx, opt, out_dtype=torch.float32, bias_grad=True)
    assert np.array_equal(gbi.cpu().numpy(), gi.double().sum(dim=0).numpy().astype(np.float32))
    # a second call on the same workspace with other data: nothing of the first call is left over
    _, _, gb2 = ops.linear_backward(gyd * 2, wd, xq, sx, opt, out_dtype=torch.float32, bias_grad=True)
    _, _, gb1 = ops.linear_backward(gyd, wd, xq, sx, opt, out_dtype=torch.float32, bias_grad=True)
    assert torch.equal(gb2, gb1 * 2)


def test_hq_linear_bias_gradient_from_fused_call(gpu, fresh_args):
    """HQ_Linear with a bias: its bias gradient comes from the fused call and equals torch's
    reduction of g_y up to the fp32 accumulation bound."""
    from hot_amd.quant_matmul import HQ_Linear
    torch.manual_seed(0)
    lin = HQ_Linear(96, 200).to(gpu)              # 200 = 8 * 25: n_o = 8
    x = torch.randn(4, 64, 96, device=gpu, requires_grad=True)
    fresh_args.batched_mode = "flatten"
    y = lin(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    ref = gy.reshape(-1, 200).double().sum(dim=0)
    assert lin.bias.grad.shape == (200,)
    assert float((lin.bias.grad.double() - ref).abs().max()) <= 256 * 2.0 ** -24 * float(gy.abs().sum(dim=(0, 1)).max())


@pytest.mark.parametrize("L", [448, 200])
def test_hq_linear_scheme_hadamard(gpu, fresh_args, L):
    """transform_scheme "hadamard" (utils/quant_matmul.py:182-183,229-230,262-263,294-295,337-339): both
    token-wise transforms are the whole block Hadamard of make_hadamard(tokens) instead of the low-rank
    projection, everything else as in gih_gwlr.  Bit-exact against the oracle configured with every
    coefficient kept, and within the tolerance against the op-for-op port of that branch."""
    from hot_amd.quant_matmul import HQ_Linear
    I, O = 96, 128
    fresh_args.transform_scheme = "hadamard"
    torch.manual_seed(1)
    lin = HQ_Linear(I, O).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    lin(x).backward(gy)
    n = orc.pow2_factor_max16(L)
    assert n == (16 if L == 448 else 8) and lin.hadamard_bs.shape == (n, n)
    assert np.array_equal(lin.hadamard_bs.cpu().numpy(), orc.hadamard(n))
    ocfg = orc.HotConfig(hla_n=n, hla_rows=tuple(range(n)))
    xq_ref, sx_ref = orc.abc_forward(x.detach().cpu().numpy(), ocfg)
    tr = orc.linear_backward(gy.cpu().numpy(), lin.weight.detach().cpu().numpy(), xq_ref, sx_ref, ocfg)
    assert np.array_equal(x.grad.cpu().numpy(), tr.g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), tr.g_w)
    h_out = torch.tensor(orc.make_hadamard(O), dtype=torch.float32)
    h_bs = torch.tensor(orc.make_hadamard(L), dtype=torch.float32)
    xq, sx = fq.setup_context(x.detach().cpu(), h_bs, fq.PortConfig())
    gi_ref, gw_ref = fq.backward(gy.cpu(), lin.weight.detach().cpu(), xq, sx, h_out, h_bs, fq.PortConfig(),
                                 scheme="hadamard")
    assert rel(x.grad.cpu().numpy(), gi_ref.numpy()) < REL_TOL
    assert rel(lin.weight.grad.cpu().numpy(), gw_ref.numpy()) < REL_TOL


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("L,O,I,rule,variant", [
    (448, 192, 160, "python", dict()),                                            # n = 64, r = 36, INT4
    (64 * 5, 208, 72, "python", dict(gx_bits=8, w_bits=8)),
    (1344, 96, 264, "python", dict(gx_round=orc.ROUND_STOCH, w_round=orc.ROUND_STOCH, seed=11)),
    (512, 256, 128, "paper", dict(w_scale=orc.SCALE_SAWB)),                       # n = 16, r = 8
    (200, 40, 24, "python", dict(gx_round=orc.ROUND_STOCH, seed=4)),              # n = 8, one ragged strip
    (49, 64, 32, "python", dict()),                                               # n = 1: nothing projected
    (384, 96, 72, "python", dict()),                                              # n = 128, r = 36: the widest block one thread holds
    (640, 64, 40, "python", dict(gx_bits=8, w_bits=8, gx_round=orc.ROUND_STOCH, seed=5)),   # n = 128, five blocks
    (768, 64, 40, "python", dict()),                                              # n = 256, r = 136: the two-level path, packed INT4
    (2048, 48, 264, "python", dict(gx_bits=8, w_bits=8)),                         # n = 2048, two channel strips of the expansion
    (3072, 32, 24, "python", dict(gx_round=orc.ROUND_STOCH, seed=9)),             # n = 1024, three blocks, stochastic
    # a step per coefficient row of P g_y (norm_quantizer, the canonical recipe's g_y quantiser)
    (448, 192, 160, "python", dict(gx_scale=orc.SCALE_ROW, gx_round=orc.ROUND_STOCH, seed=6)),
    (384, 96, 72, "python", dict(gx_scale=orc.SCALE_ROW, gx_bits=8, w_bits=8)),    # n = 128
    (512, 256, 128, "paper", dict(gx_scale=orc.SCALE_ROW, gx_round=orc.ROUND_STOCH, w_scale=orc.SCALE_SAWB, seed=2)),
])
def test_gx_lowrank_matches_oracle(gpu, dtype, L, O, I, rule, variant):
    """g_x of the schemes "low_rank" / "gilr_gwh" (hot_gx_lowrank): the projected g_y stored untransposed,
    W quantised without a transform, the product in fp32 and the expansion pass, bit for bit the oracle."""
    from hot_amd import ops
    x, w, gy = make_case(L, O, I, seed=L + I, dtype=dtype)
    ocfg, opt = both_configs(L, rule=rule, max_block=8192, **variant)
    assert ocfg.hla_n == (16 if rule == "paper" else orc.hla_rows(L)[0])
    gx = ops.gx_lowrank(gy.to(gpu), w.to(gpu), opt)
    tr = orc.gx_lowrank(gy.float().numpy(), w.float().numpy(), ocfg)
    assert gx.dtype == dtype and tuple(gx.shape) == (L, I)
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dtype))


def test_gx_lowrank_refuses_what_it_cannot_do(gpu):
    from hot_amd import ops
    x, w, gy = make_case(256, 64, 32, seed=0)
    _, opt = both_configs(256, gx_scale=orc.SCALE_SAWB)
    with pytest.raises(ops.HotError, match="absmax steps"):
        ops.gx_lowrank(gy.to(gpu), w.to(gpu), opt)
    n, rows = orc.hla_rows(256)
    big = ops.HotOptions(hla_n=n, hla_rows=tuple(int(v) for v in rows), gx_scale=orc.SCALE_ROW)
    with pytest.raises(ops.HotError, match="token blocks up to 128"):
        ops.gx_lowrank(gy.to(gpu), w.to(gpu), big)
    n, rows = orc.hla_rows(128)
    odd = ops.HotOptions(hla_n=n, hla_rows=tuple(int(v) for v in rows))
    with pytest.raises(ops.HotError, match="not a multiple of hla_n"):
        ops.gx_lowrank(gy[:192].to(gpu), w.to(gpu), odd)


@pytest.mark.parametrize("scheme", ["low_rank", "gilr_gwh"])
@pytest.mark.parametrize("L", [448, 200, 384, 512])
def test_hq_linear_lowrank_gx_schemes(gpu, fresh_args, scheme, L):
    """transform_scheme "low_rank" (utils/quant_matmul.py:184-185,231-232,263-264,296-297,334-335) and
    "gilr_gwh" (:186-187,233-234,265-266,298-299,336-338) through HQ_Linear: g_x by projection along the
    tokens and expansion, g_W as in gih_gwlr / hadamard.  Bit-exact against the oracle, within the
    tolerance against the op-for-op port of those branches."""
    from hot_amd.quant_matmul import HQ_Linear
    I, O = 96, 128
    fresh_args.transform_scheme = scheme
    torch.manual_seed(2)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    lin(x).backward(gy)
    xn, gyn, wn = x.detach().cpu().numpy(), gy.cpu().numpy(), lin.weight.detach().cpu().numpy()
    n_lr, rows_lr = orc.hla_rows(L)                      # 64 / 36 at 448, 8 / 5 at 200, 128 / 36 at 384, 512 / 136 at 512
    cfg_gx = orc.HotConfig(hla_n=n_lr, hla_rows=tuple(int(v) for v in rows_lr))
    if scheme == "low_rank":
        cfg_gw = cfg_gx
        h_out = torch.zeros(1, 1)
        h_bs = torch.tensor(orc.make_WHT(L), dtype=torch.float32)
    else:
        n16 = orc.pow2_factor_max16(L)
        cfg_gw = orc.HotConfig(hla_n=n16, hla_rows=tuple(range(n16)))
        h_out = torch.tensor(orc.make_WHT(L), dtype=torch.float32)
        h_bs = torch.tensor(orc.make_hadamard(L), dtype=torch.float32)
    xq_ref, sx_ref = orc.abc_forward(xn, cfg_gw)
    assert np.array_equal(x.grad.cpu().numpy(), orc.gx_lowrank(gyn, wn, cfg_gx).g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), orc.linear_backward(gyn, wn, xq_ref, sx_ref, cfg_gw).g_w)
    xq, sx = fq.setup_context(x.detach().cpu(), h_bs, fq.PortConfig())
    gi_ref, gw_ref = fq.backward(gy.cpu(), lin.weight.detach().cpu(), xq, sx, h_out, h_bs, fq.PortConfig(), scheme=scheme)
    assert rel(x.grad.cpu().numpy(), gi_ref.numpy()) < REL_TOL
    assert rel(lin.weight.grad.cpu().numpy(), gw_ref.numpy()) < REL_TOL


def test_hq_linear_lowrank_with_per_token_quantisers(gpu, fresh_args):
    """transform_scheme "low_rank" under the quantisers of the reference's canonical recipe for g_y
    (quantBWDGogi = quantBWDGogw = "nq": a step per row of the quantised matrix, stochastic rounding,
    utils/quant_matmul.py:19-37,244-255,307-318): the projected g_y [L', O] takes a step per coefficient row
    on the g_x side, (P g_y)^T a step per channel on the g_W side.  Bit-exact against the oracle."""
    from hot_amd.quant_matmul import HQ_Linear
    L, I, O = 448, 96, 128
    fresh_args.transform_scheme = "low_rank"
    fresh_args.quantBWDGogi = fresh_args.quantBWDGogw = "nq"
    torch.manual_seed(12)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    step = fresh_args.sr_step
    lin(x).backward(gy)
    xn, gyn, wn = x.detach().cpu().numpy(), gy.cpu().numpy(), lin.weight.detach().cpu().numpy()
    seed = (int(fresh_args.sr_seed) << 20) + step
    ocfg, _ = both_configs(L, seed=seed, gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
                           gw_scale=orc.SCALE_ROW)
    xq_ref, sx_ref = orc.abc_forward(xn, ocfg)
    assert np.array_equal(x.grad.cpu().numpy(), orc.gx_lowrank(gyn, wn, ocfg).g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), orc.linear_backward(gyn, wn, xq_ref, sx_ref, ocfg).g_w)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("L,O,I,variant", [
    (448, 192, 160, dict(seed=1)),
    (1000, 208, 72, dict(seed=2, w_scale=orc.SCALE_SAWB)),          # K padded from 208 to 256 in both planes
    (197, 80, 264, dict(seed=3, w_round=orc.ROUND_STOCH)),
    (4096, 768, 512, dict(seed=4)),
])
def test_gx_luq_matches_oracle(gpu, dtype, L, O, I, variant):
    """g_x with the logarithmic quantiser on g_y (hot_gx_luq): codes 0 / +-2^j as two INT8 planes against
    [16 w | w], bit for bit the oracle (same uniforms, same float operations)."""
    from hot_amd import ops
    x, w, gy = make_case(L, O, I, seed=L + O, dtype=dtype)
    ocfg = orc.HotConfig(**variant)
    opt = ops.HotOptions(n_o=ocfg.n_o, w_round=ocfg.w_round, w_scale=ocfg.w_scale, seed=ocfg.seed)
    gx = ops.gx_luq(gy.to(gpu), w.to(gpu), opt)
    tr = orc.gx_luq(gy.float().numpy(), w.float().numpy(), ocfg)
    assert int(np.abs(tr.qG).max()) >= 128                           # the top level is in use
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tail", [10.0, 1000.0])
def test_gx_luq_negative_tail_beyond_the_maximum(gpu, dtype, tail):
    """The step of the logarithmic quantiser comes from the MAXIMUM of the transformed tensor
    (utils/quant_matmul.py:60-61), so negative elements beyond it take larger codes; the two-plane
    product holds them at -2^10 (a stated deviation, restated by the oracle's gx_luq).  Whole blocks of
    g_y at -tail x the largest entry put such elements into the transform."""
    from hot_amd import ops
    L, O, I = 448, 192, 160
    x, w, gy = make_case(L, O, I, seed=77, dtype=torch.float32)
    top = float(gy.abs().max())
    gy[5, 32:48] = -tail * top
    gy[200, 0:16] = -tail * top * 0.37
    gy[447, 176:192] = tail * top * 1e-3            # positive side: nothing special
    gy, w = gy.to(dtype), w.to(dtype)
    ocfg = orc.HotConfig(seed=6)
    opt = ops.HotOptions(n_o=ocfg.n_o, seed=ocfg.seed)
    gx = ops.gx_luq(gy.to(gpu), w.to(gpu), opt)
    tr = orc.gx_luq(gy.float().numpy(), w.float().numpy(), ocfg)
    free = orc.gx_luq(gy.float().numpy(), w.float().numpy(), ocfg, max_exp=None)
    assert int(np.abs(tr.qG).max()) == 1024 and int(np.abs(free.qG).max()) > 1024      # the bound is active
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dtype))


def test_hq_linear_with_luq_on_the_gx_path(gpu, fresh_args):
    """quantBWDGogi = "luq" through HQ_Linear: g_x from hot_gx_luq, g_W as with any other setting."""
    from hot_amd.quant_matmul import HQ_Linear
    L, I, O = 448, 96, 128
    fresh_args.quantBWDGogi = "luq"
    torch.manual_seed(3)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    step = fresh_args.sr_step
    lin(x).backward(gy)
    xn, gyn, wn = x.detach().cpu().numpy(), gy.cpu().numpy(), lin.weight.detach().cpu().numpy()
    seed = (int(fresh_args.sr_seed) << 20) + step
    ocfg, _ = both_configs(L, seed=seed)
    xq_ref, sx_ref = orc.abc_forward(xn, ocfg)
    assert np.array_equal(x.grad.cpu().numpy(), orc.gx_luq(gyn, wn, ocfg).g_x)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), orc.linear_backward(gyn, wn, xq_ref, sx_ref, ocfg).g_w)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("L,O,I,rule,variant", [
    (448, 192, 160, "python", dict(seed=1)),                       # n = 64, r = 36
    (1576, 80, 264, "python", dict(seed=2, act_bits=4)),            # n = 8: L' is no multiple of 8, rows padded
    (512, 256, 128, "paper", dict(seed=3)),                        # n = 16, r = 8
    (197, 40, 24, "python", dict(seed=4)),                         # n = 1: nothing projected, 197 -> 200 per row
    (4096, 768, 512, "python", dict(seed=5)),
])
def test_gw_luq_matches_oracle(gpu, dtype, L, O, I, rule, variant):
    """g_W with the logarithmic quantiser on the projected g_y (hot_gw_luq): the projection in fp32 by
    the canonical butterflies, codes 0 / +-2^j as two INT8 planes against the activation buffer, the
    integer sums combined: bit for bit the oracle (same uniforms, same float operations)."""
    from hot_amd import ops
    x, w, gy = make_case(L, O, I, seed=L + O, dtype=dtype)
    ocfg, opt = both_configs(L, rule=rule, gw_bits=4, **variant)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    xq_ref, sx_ref = orc.abc_forward(x.float().numpy(), ocfg)
    gw = ops.gw_luq(gy.to(gpu), xq, sx, opt)
    ref = orc.gw_luq(gy.float().numpy(), xq_ref, sx_ref, ocfg)
    assert gw.dtype == dtype and tuple(gw.shape) == (O, I)
    assert torch.equal(gw.cpu(), torch.from_numpy(ref).to(dtype))


def test_gw_luq_refuses_what_it_cannot_do(gpu):
    from hot_amd import ops
    x, w, gy = make_case(256, 64, 32, seed=0)
    _, opt = both_configs(256)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    with pytest.raises(ops.HotError, match="4 bits"):
        ops.gw_luq(gy.to(gpu), xq, sx, opt)                        # gw_bits = 8


@pytest.mark.parametrize("how", ["flag", "auto"])
def test_hq_linear_with_luq_on_the_gw_path(gpu, fresh_args, how):
    """quantBWDGogw = "luq" at GogwQuantBit = 4, and luq_quantizer picked for both products of a layer
    under quantAuto (where the g_W branch reads GogiQuantBit, utils/quant_matmul.py:307-308): g_W through
    hot_gw_luq, g_x by the fused call or hot_gx_luq.  Bit-exact against the oracle."""
    from hot_amd.quant_matmul import HQ_Linear
    L, I, O = 448, 96, 128
    torch.manual_seed(6)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    lin.layer_name = "blk.fc"
    if how == "flag":
        fresh_args.quantBWDGogw = "luq"
        fresh_args.GogwQuantBit = 4
    else:
        fresh_args.quantAuto = True
        fresh_args.layer_quant_dict = {"blk.fc_gx": "luq_quantizer", "blk.fc_gw": "luq_quantizer"}
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    step = fresh_args.sr_step
    lin(x).backward(gy)
    xn, gyn, wn = x.detach().cpu().numpy(), gy.cpu().numpy(), lin.weight.detach().cpu().numpy()
    seed = (int(fresh_args.sr_seed) << 20) + step
    ocfg, _ = both_configs(L, seed=seed, gw_bits=4, gw_round=orc.ROUND_STOCH)
    xq_ref, sx_ref = orc.abc_forward(xn, ocfg)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), orc.gw_luq(gyn, xq_ref, sx_ref, ocfg))
    gx_ref = orc.gx_luq(gyn, wn, ocfg).g_x if how == "auto" else orc.linear_backward(gyn, wn, xq_ref, sx_ref, ocfg).g_x
    assert np.array_equal(x.grad.cpu().numpy(), gx_ref)


@pytest.mark.parametrize("path,T", [("luq", 64), ("luq", 197), ("low_rank", 64), ("gilr_gwh", 48), ("low_rank", 256)])
def test_hq_linear_3d_per_sample_on_the_separate_gx_paths(gpu, fresh_args, path, T):
    """3-D activations with a step per sample (the reference's vmap over the batch,
    utils/quant_matmul.py:79-83,118-122) through quantBWDGogi = "luq" and the schemes that project g_y
    along the tokens: every sample is the 2-D case of its own tokens, sample b seeded with seed + b,
    the weight gradients added in fp32 in sample order.  Against the oracle, sample by sample."""
    from hot_amd.quant_matmul import HQ_Linear
    B, I, O = 3, 96, 128
    fresh_args.batched_mode = "per_sample"
    if path == "luq":
        fresh_args.quantBWDGogi = "luq"
    else:
        fresh_args.transform_scheme = path
    torch.manual_seed(T)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(B, T, I, device=gpu, requires_grad=True)
    gy = torch.randn(B, T, O, device=gpu) * 1e-3 * (10.0 ** torch.arange(B, device=gpu).float().view(B, 1, 1))
    step = fresh_args.sr_step
    lin(x).backward(gy)
    wn = lin.weight.detach().cpu().numpy()
    seed = (int(fresh_args.sr_seed) << 20) + step
    n_lr, rows_lr = orc.hla_rows(T)
    gxs, gw = [], None
    for b in range(B):
        cfg_gx = orc.HotConfig(hla_n=n_lr, hla_rows=tuple(int(v) for v in rows_lr), seed=seed + b)
        if path == "gilr_gwh":
            n16 = orc.pow2_factor_max16(T)
            cfg_gw = orc.HotConfig(hla_n=n16, hla_rows=tuple(range(n16)), seed=seed + b)
        else:
            cfg_gw = cfg_gx
        xn, gyn = x[b].detach().cpu().numpy(), gy[b].cpu().numpy()
        xq_ref, sx_ref = orc.abc_forward(xn, cfg_gw)
        gw_b = orc.linear_backward(gyn, wn, xq_ref, sx_ref, cfg_gw).g_w
        gw = gw_b if gw is None else (gw + gw_b).astype(np.float32)
        gxs.append(orc.gx_luq(gyn, wn, cfg_gx).g_x if path == "luq" else orc.gx_lowrank(gyn, wn, cfg_gx).g_x)
    assert np.array_equal(x.grad.cpu().numpy(), np.stack(gxs))
    assert np.array_equal(lin.weight.grad.cpu().numpy(), gw)


def test_hq_linear_under_autocast_matches_the_inline_buffer_write(gpu, fresh_args):
    """The reference trains under autocast (ViT_main.py:386): x stays fp32, F.linear makes and releases
    a bf16 copy of it while the buffer kernels run on the side stream.  Their outputs and workspace come
    from the side stream's own pool, so the released copy cannot be handed to them; the buffer, g_x and
    g_W equal those of the same step with the buffer written in line, over several layers in a row."""
    from hot_amd import quant_matmul as qm
    L, I, O = 3200, 256, 512
    torch.manual_seed(4)
    lins = [qm.HQ_Linear(I, O).to(gpu), qm.HQ_Linear(O, I).to(gpu), qm.HQ_Linear(I, O).to(gpu)]
    x0 = torch.randn(L, I, device=gpu)
    gy = torch.randn(L, O, device=gpu) * 1e-3

    def run(overlap):
        qm.overlap_buffer_write = overlap
        fresh_args.sr_step = 0
        for m in lins:
            m.zero_grad(set_to_none=True)
        x = x0.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            h = x
            for m in lins:
                h = m(h).float()                    # fp32 activations between the layers, as x is
        h.backward(gy)
        torch.cuda.synchronize()
        return [x.grad.clone()] + [m.weight.grad.clone() for m in lins] + [m.bias.grad.clone() for m in lins]

    try:
        ref = run(False)
        for _ in range(3):
            got = run(True)
            for a, b in zip(got, ref):
                assert torch.equal(a, b)
    finally:
        qm.overlap_buffer_write = True


@pytest.mark.parametrize("gw_bits,act_bits", [(4, 8), (4, 4), (8, 4)])
@pytest.mark.parametrize("path", ["luq", "low_rank"])
def test_hq_linear_gw_widths_on_the_separate_gx_paths(gpu, fresh_args, path, gw_bits, act_bits):
    """quantBWDGogi = "luq" and transform_scheme = "low_rank" compute g_W by the token-wise kernel and an
    INT8 product of byte codes, whatever GogwQuantBit / actQuantBit are (utils/quant_matmul.py:307-324:
    4-bit codes are integers in [-7, 7] all the same): every width pair against the oracle."""
    from hot_amd.quant_matmul import HQ_Linear
    L, I, O = 448, 96, 128
    fresh_args.GogwQuantBit, fresh_args.actQuantBit = gw_bits, act_bits
    if path == "luq":
        fresh_args.quantBWDGogi = "luq"
    else:
        fresh_args.transform_scheme = "low_rank"
    torch.manual_seed(9)
    lin = HQ_Linear(I, O, bias=False).to(gpu)
    x = torch.randn(L, I, device=gpu, requires_grad=True)
    gy = torch.randn(L, O, device=gpu) * 1e-3
    step = fresh_args.sr_step
    lin(x).backward(gy)
    xn, gyn, wn = x.detach().cpu().numpy(), gy.cpu().numpy(), lin.weight.detach().cpu().numpy()
    seed = (int(fresh_args.sr_seed) << 20) + step
    ocfg, _ = both_configs(L, seed=seed, gw_bits=gw_bits, act_bits=act_bits)
    xq_ref, sx_ref = orc.abc_forward(xn, ocfg)
    assert int(np.abs(xq_ref).max()) == (7 if act_bits == 4 else 127)
    tr = orc.linear_backward(gyn, wn, xq_ref, sx_ref, ocfg)
    assert int(np.abs(tr.qGp).max()) == (7 if gw_bits == 4 else 127)
    assert np.array_equal(lin.weight.grad.cpu().numpy(), tr.g_w)
    gx_ref = orc.gx_luq(gyn, wn, ocfg).g_x if path == "luq" else orc.gx_lowrank(gyn, wn, ocfg).g_x
    assert np.array_equal(x.grad.cpu().numpy(), gx_ref)


@pytest.mark.parametrize("variant", [dict(), dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW,
                                                 gw_round=orc.ROUND_STOCH, gw_scale=orc.SCALE_ROW, seed=3)])
def test_backward_fp16(gpu, variant):
    """fp16 tensors (the reference's op dispatches them, cuda_measure/HLQ_backward_kernel.cu:474-515): the
    codes and steps are those of the oracle on the fp16 values, the outputs its fp32 results rounded once."""
    L, O, I = 448, 192, 160
    x, w, gy = make_case(L, O, I, seed=21, dtype=torch.float16)
    ocfg, opt = both_configs(L, **variant)
    gx, gw, tr = run_both(x, w, gy, ocfg, opt, gpu)
    assert gx.dtype == torch.float16 and gw.dtype == torch.float16
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(torch.float16))
    assert torch.equal(gw.cpu(), torch.from_numpy(tr.g_w).to(torch.float16))
