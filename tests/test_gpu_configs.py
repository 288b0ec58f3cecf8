"""The benchmark configurations at their own size, through the C ABI, against the CPU oracle.

  * the four ViT-B layer shapes at 64 x 197 tokens, fp32 and bf16, quantiser variants; two of them as
    [64, 197, C] activations with per-sample steps (the reference's own treatment of a batch);
  * the kernel-level sweep of the row-wise Hadamard quantiser (M up to 65536, K up to 11008, per-channel
    scales drawn log-uniform), oracle on sampled rows: rows are independent under per-token steps;
  * the Llama-7B shapes at 8192 tokens with heavy-tailed (Student-t) gradient columns: steps of the
    whole tensors, codes and final gradients on sampled rows and columns that touch every output tile;
  * one step of the whole ViT-B/16 with every layer swapped.

Integer stages and step sizes are compared bit for bit; final gradients equal the oracle's after the
same rounding to the output type."""
import numpy as np
import pytest
import torch

from oracle import hot_oracle as orc

pytestmark = pytest.mark.gpu

F32 = np.float32


def vit_inputs(L, O, I, dtype, seed):
    """x ~ N(0, 1); g_y ~ N(0, 1e-3) with 1 % of the entries x 50; W uniform(+-1/sqrt(I))."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(L, I, generator=g).to(dtype)
    w = ((torch.rand(O, I, generator=g) * 2 - 1) / I ** 0.5).to(dtype)
    gy = torch.randn(L, O, generator=g) * 1e-3
    gy = torch.where(torch.rand(L, O, generator=g) < 0.01, gy * 50, gy).to(dtype)
    return x, w, gy


def options_pair(ocfg):
    from hot_amd import ops
    return ops.HotOptions(n_o=ocfg.n_o, hla_n=ocfg.hla_n, hla_rows=ocfg.hla_rows, gx_bits=ocfg.gx_bits,
                          w_bits=ocfg.w_bits, gw_bits=ocfg.gw_bits, act_bits=ocfg.act_bits, gx_round=ocfg.gx_round,
                          w_round=ocfg.w_round, gw_round=ocfg.gw_round, act_round=ocfg.act_round,
                          gx_scale=ocfg.gx_scale, w_scale=ocfg.w_scale, gw_scale=ocfg.gw_scale,
                          act_scale=ocfg.act_scale, seed=ocfg.seed)


VIT_SHAPES = {"qkv": (2304, 768), "proj": (768, 768), "fc1": (3072, 768), "fc2": (768, 3072)}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layer", ["qkv", "proj", "fc1", "fc2"])
def test_vit_b_layers_full_size(gpu, layer, dtype):
    """L = 12608 tokens (batch 64 x 197), HQ INT4 g_x + HLA (n = 64, r = 36) INT8 g_W, nearest, per tensor."""
    from hot_amd import ops
    L = 12608
    O, I = VIT_SHAPES[layer]
    x, w, gy = vit_inputs(L, O, I, dtype, seed=O + I)
    ocfg = orc.HotConfig.python_rule(L)
    assert (ocfg.hla_n, len(ocfg.hla_rows)) == (64, 36)
    opt = options_pair(ocfg)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    gx, gw = ops.linear_backward(gy.to(gpu), w.to(gpu), xq, sx, opt)
    xq_ref, sx_ref = orc.abc_forward(x.float().numpy(), ocfg)
    tr = orc.linear_backward(gy.float().numpy(), w.float().numpy(), xq_ref, sx_ref, ocfg)
    lp = xq_ref.shape[0]
    got_xq = xq.cpu().numpy()
    assert np.array_equal(got_xq[:, :lp], xq_ref.T) and not got_xq[:, lp:].any()
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dtype))
    assert torch.equal(gw.cpu(), torch.from_numpy(tr.g_w).to(dtype))


@pytest.mark.parametrize("layer,dtype,variant", [
    ("qkv", torch.bfloat16, dict(gx_bits=8, w_bits=8, gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, seed=11)),
    ("fc2", torch.bfloat16, dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
                                 gw_scale=orc.SCALE_ROW, w_scale=orc.SCALE_SAWB, act_scale=orc.SCALE_SAWB, seed=5)),
    ("proj", torch.float32, dict(gx_scale=orc.SCALE_ROW, gw_scale=orc.SCALE_ROW, gx_bits=8, w_bits=8)),
    ("fc1", torch.bfloat16, dict(rule="paper", gx_round=orc.ROUND_STOCH, gw_round=orc.ROUND_STOCH, seed=3)),
])
def test_vit_b_layers_full_size_quantiser_variants(gpu, layer, dtype, variant):
    """INT8 / stochastic / per-token / SAWB variants and the n = 16, r = 8 low-rank setting at 12608 tokens."""
    from hot_amd import ops
    L = 12608
    O, I = VIT_SHAPES[layer]
    variant = dict(variant)
    rule = variant.pop("rule", "python")
    x, w, gy = vit_inputs(L, O, I, dtype, seed=7 + O)
    ocfg = orc.HotConfig.python_rule(L, **variant) if rule == "python" else orc.HotConfig.paper(16, 8, **variant)
    opt = options_pair(ocfg)
    xq, sx = ops.abc_forward(x.to(gpu), opt)
    gx, gw = ops.linear_backward(gy.to(gpu), w.to(gpu), xq, sx, opt)
    xq_ref, sx_ref = orc.abc_forward(x.float().numpy(), ocfg)
    tr = orc.linear_backward(gy.float().numpy(), w.float().numpy(), xq_ref, sx_ref, ocfg)
    assert np.array_equal(xq.cpu().numpy()[:, :xq_ref.shape[0]], xq_ref.T)
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    assert torch.equal(gx.cpu(), torch.from_numpy(tr.g_x).to(dtype))
    assert torch.equal(gw.cpu(), torch.from_numpy(tr.g_w).to(dtype))


# ------------------------------------------------------------ kernel-level sweep of the row-wise quantiser

@pytest.mark.parametrize("layer,variant", [
    ("proj", dict()),
    ("qkv", dict(gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH, seed=5)),
])
def test_vit_b_layers_per_sample_steps(gpu, layer, variant):
    """The reference's own treatment of the ViT batch: [64, 197, C] activations, every sample with steps
    of its own (197 tokens: one-token blocks, nothing projected), through the batched entry points at
    the layer's real size; activation buffer, g_x and the summed g_W against the oracle, bf16."""
    from hot_amd import ops
    O, I = VIT_SHAPES[layer]
    B, T = 64, 197
    x, w, gy = vit_inputs(B * T, O, I, torch.bfloat16, seed=O + I + 1)
    g = torch.Generator().manual_seed(3)
    mag = (10.0 ** (torch.rand(B, 1, 1, generator=g) * 2 - 1)).to(torch.bfloat16)        # samples of different size
    x3, gy3 = x.reshape(B, T, I), (gy.reshape(B, T, O) * mag).contiguous()
    ocfg = orc.HotConfig.python_rule(T, **variant)
    assert ocfg.hla_n == 1
    opt = options_pair(ocfg)
    xq, sx = ops.abc_forward_batched(x3.to(gpu), opt)
    gx, gw = ops.linear_backward_batched(gy3.to(gpu), w.to(gpu), xq, sx, opt)
    ranges = ops.backward_batched_ranges(B, T, O, I, opt)
    xq_ref, sx_ref = orc.abc_forward_batched(x3.float().numpy(), ocfg)
    gx_ref, gw_ref, _ = orc.linear_backward_batched(gy3.float().numpy(), w.float().numpy(), xq_ref, sx_ref, ocfg,
                                                    gw_ranges=ranges)
    kg = ops.kpad_group(T, opt)
    got = xq.cpu().numpy().reshape(I, B, kg)
    assert np.array_equal(got[:, :, :T], xq_ref.transpose(2, 0, 1)) and not got[:, :, T:].any()
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    assert torch.equal(gx.cpu(), torch.from_numpy(gx_ref).to(torch.bfloat16))
    assert torch.equal(gw.cpu(), torch.from_numpy(gw_ref).to(torch.bfloat16))


@pytest.mark.parametrize("M", [4096, 16384, 65536])
@pytest.mark.parametrize("K", [768, 3072, 4096, 11008])
def test_hq_rowwise_sweep_sizes(gpu, M, K):
    """bf16 input ~ N(0, 1) x per-channel scale 10^U(-1, 1); Hadamard blocks 16 / 32 / 64; INT4-packed
    and INT8 codes + per-token fp32 steps; sampled rows (first, last, around the middle, random)."""
    from hot_amd import ops
    g = torch.Generator(device=gpu).manual_seed(M + K)
    x = (torch.randn(M, K, generator=g, device=gpu) *
         (10.0 ** (torch.rand(K, generator=g, device=gpu) * 2 - 1))).to(torch.bfloat16)
    rows = np.unique(np.concatenate([[0, 1, M // 2 - 1, M // 2, M - 2, M - 1],
                                     np.random.default_rng(K).integers(0, M, 58)]))
    xs = x[torch.from_numpy(rows).to(gpu)].float().cpu().numpy()
    for n in (16, 32, 64):
        t = orc.fwht_blocks_last(xs, n)
        for bits in (4, 8):
            q_ref, s_ref = orc.quant(t, bits, orc.SCALE_ROW)
            codes, s = ops.hq_rowwise(x, n=n, bits=bits, rounding="nearest", scale="row")
            got = codes[torch.from_numpy(rows).to(gpu)].cpu().numpy()
            got = orc.unpack_int4(got)[:, :K] if bits == 4 else got[:, :K]
            assert np.array_equal(s.cpu().numpy()[rows], s_ref), (n, bits)
            assert np.array_equal(got, q_ref), (n, bits)
    # stochastic rounding at this size: element indices up to M * K (7.2e8 at the largest case)
    q_ref, s_ref = orc.quant(orc.fwht_blocks_last(xs, 16), 4, orc.SCALE_ROW, orc.ROUND_STOCH, seed=9, stream=orc.STREAM_GX,
                             index=(rows.astype(np.int64)[:, None] * K + np.arange(K, dtype=np.int64)[None, :]))
    codes, s = ops.hq_rowwise(x, n=16, bits=4, rounding="stoch", scale="row", seed=9)
    got = orc.unpack_int4(codes[torch.from_numpy(rows).to(gpu)].cpu().numpy())[:, :K]
    assert np.array_equal(s.cpu().numpy()[rows], s_ref) and np.array_equal(got, q_ref)


# ------------------------------------------------------------ Llama-7B shapes, heavy-tailed gradient columns

def llama_inputs(L, O, I, seed):
    """bf16; W random-init; g_y ~ N(0, 1e-3) with 0.5 % of its columns replaced by Student-t (nu = 3)
    draws at the same scale (outlier channels with heavy tails)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(L, I, generator=g)
    w = (torch.rand(O, I, generator=g) * 2 - 1) / I ** 0.5
    gy = torch.randn(L, O, generator=g) * 1e-3
    cols = torch.randperm(O, generator=g)[: max(1, O // 200)]
    z = torch.randn(L, len(cols), generator=g)
    chi = (torch.randn(L, len(cols), 3, generator=g) ** 2).sum(dim=-1)
    gy[:, cols] = z / torch.sqrt(chi / 3.0) * 1e-3
    return x.to(torch.bfloat16), w.to(torch.bfloat16), gy.to(torch.bfloat16), cols.numpy()


@pytest.mark.parametrize("O,I", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_llama_layers_full_size(gpu, O, I):
    """q/k/v/o, gate/up and down at 8192 tokens, HQ INT4 g_x + HLA n = 16 / r = 8 INT8 g_W.  The oracle
    runs every transform and quantiser on the whole tensors (steps of the whole tensors, every code of
    W, of the activation buffer and of both g_y operands); the two large products are evaluated on
    sampled rows and columns of g_x and g_W that together touch every output tile."""
    from hot_amd import ops
    L = 8192
    x, w, gy, heavy = llama_inputs(L, O, I, seed=O + I)
    ocfg = orc.HotConfig.paper(16, 8)
    opt = options_pair(ocfg)
    xd, wd, gyd = x.to(gpu), w.to(gpu), gy.to(gpu)
    xq, sx = ops.abc_forward(xd, opt)
    gx, gw = ops.linear_backward(gyd, wd, xq, sx, opt)
    # the three quantise kernels on their own, for codes and steps
    qg_d, sg_d = ops.hq_rowwise(gyd, n=16, bits=4)
    qgp_d, sgp_d, lp = ops.hla_tokenwise(gyd, 16, list(ocfg.hla_rows), bits=8)
    qw_d, sw_d = ops.wq_colwise(wd, n=16, bits=4)
    torch.cuda.synchronize()

    gyn, wn, xn = gy.float().numpy(), w.float().numpy(), x.float().numpy()
    rows_sel = np.asarray(ocfg.hla_rows)
    xq_ref, sx_ref = orc.abc_forward(xn, ocfg)                                   # [L', I]
    assert lp == xq_ref.shape[0] == L // 2
    assert np.array_equal(xq.cpu().numpy()[:, :lp], xq_ref.T) and np.array_equal(sx.cpu().numpy(), sx_ref)
    G = orc.fwht_blocks_last(gyn, 16)
    qG, sG = orc.quant(G, 4, orc.SCALE_TENSOR)
    del G
    assert np.array_equal(sg_d.cpu().numpy(), sG)
    assert np.array_equal(orc.unpack_int4(qg_d.cpu().numpy())[:, :O], qG)
    Wh = orc.fwht_blocks_first(wn, 16)
    qW, sW = orc.quant(Wh, 4, orc.SCALE_TENSOR)                                  # [O, I]
    del Wh
    assert np.array_equal(sw_d.cpu().numpy(), sW)
    assert np.array_equal(orc.unpack_int4(qw_d.cpu().numpy())[:, :O], qW.T)
    GpT = np.ascontiguousarray(orc.fwht_blocks_first(gyn, 16, rows_sel).T)       # [O, L']
    qGp, sGp = orc.quant(GpT, 8, orc.SCALE_TENSOR)
    del GpT
    assert np.array_equal(sgp_d.cpu().numpy(), sGp)
    got = qgp_d.cpu().numpy()
    assert np.array_equal(got[:, :lp], qGp) and not got[:, lp:].any()
    # the heavy-tailed columns are what sets the steps: the largest coefficient sits in one of their blocks
    assert np.abs(gyn[:, heavy]).max() > 8 * np.abs(np.delete(gyn, heavy, axis=1)).max()

    rng = np.random.default_rng(O)
    def sample(n):
        return np.unique(np.concatenate([[0, 255, 256, n - 1], rng.integers(0, n, 28)]))
    def deq(acc, sa, sb, div):
        return torch.from_numpy((((acc.astype(F32) * F32(sa)).astype(F32) * F32(sb)).astype(F32) / F32(div)).astype(F32)
                                ).to(torch.bfloat16)
    f32 = lambda a: a.astype(np.float32)            # INT4 products: partial sums below 2^24, exact in fp32
    gx_c, gw_c = gx.cpu(), gw.cpu()
    r, c = sample(L), sample(I)
    assert torch.equal(gx_c[r], deq(f32(qG[r]) @ f32(qW), sG[0], sW[0], 16))
    assert torch.equal(gx_c[:, c], deq(f32(qG) @ f32(qW[:, c]), sG[0], sW[0], 16))
    r, c = sample(O), sample(I)
    f64 = lambda a: a.astype(np.float64)
    xqT = xq_ref                                                                # [L', I]
    assert torch.equal(gw_c[r], deq(np.rint(f64(qGp[r]) @ f64(xqT)), sGp[0], sx_ref[0], 16))
    assert torch.equal(gw_c[:, c], deq(np.rint(f64(qGp) @ f64(xqT[:, c])), sGp[0], sx_ref[0], 16))


def _hla_in_strips(a, n, rows, strip=1024):
    """fwht_blocks_first(a, n, rows) evaluated strip by strip of channels (the columns are independent):
    the same arithmetic without a second and third copy of the whole tensor."""
    out = np.empty(((a.shape[0] // n) * len(rows), a.shape[1]), dtype=F32)
    for c0 in range(0, a.shape[1], strip):
        out[:, c0:c0 + strip] = orc.fwht_blocks_first(np.ascontiguousarray(a[:, c0:c0 + strip]), n, rows)
    return out


@pytest.mark.parametrize("O,I", [(11008, 4096), (4096, 11008)])
def test_llama_layers_full_size_reference_rule(gpu, O, I):
    """Llama-7B gate/up and down at 8192 tokens with the reference's own low-rank rule
    (utils/hadamard_matmul.py:209-226: 8192 tokens -> one block of n = 8192, r = 2080 kept sequencies),
    bf16, Student-t gradient columns: the two-level token-wise path over every channel strip of the full
    widths.  Steps of the whole tensors, every code of the activation buffer and of (P g_y)^T, g_W and
    g_x on sampled rows and columns that touch every output tile."""
    from hot_amd import ops
    from hot_amd.hadamard_matmul import run_major
    L = 8192
    x, w, gy, heavy = llama_inputs(L, O, I, seed=O + I + 1)
    ocfg = orc.HotConfig.python_rule(L)
    assert (ocfg.hla_n, len(ocfg.hla_rows)) == (8192, 2080)
    if O == 11008:
        # gate/up with the rows run by run, as the layers list them for large blocks (the K order of both
        # g_W operands; g_W itself does not depend on it); down with the reference's sequency order
        ocfg.hla_rows = tuple(int(v) for v in run_major(ocfg.hla_rows))
    opt = options_pair(ocfg)
    xd, wd, gyd = x.to(gpu), w.to(gpu), gy.to(gpu)
    xq, sx = ops.abc_forward(xd, opt)
    gx, gw = ops.linear_backward(gyd, wd, xq, sx, opt)
    qgp_d, sgp_d, lp = ops.hla_tokenwise(gyd, ocfg.hla_n, list(ocfg.hla_rows), bits=8)
    torch.cuda.synchronize()
    assert lp == 2080
    rows_sel = np.asarray(ocfg.hla_rows)
    gyn, wn, xn = gy.float().numpy(), w.float().numpy(), x.float().numpy()
    # activation buffer: every code, the step
    xq_ref, sx_ref = orc.quant(_hla_in_strips(xn, L, rows_sel), 8, orc.SCALE_TENSOR)          # [L', I]
    got = xq.cpu().numpy()
    assert np.array_equal(sx.cpu().numpy(), sx_ref)
    assert np.array_equal(got[:, :lp], xq_ref.T) and not got[:, lp:].any()
    # (P g_y)^T: every code of every channel strip, the step of the whole tensor
    GpT = np.ascontiguousarray(_hla_in_strips(gyn, L, rows_sel).T)                           # [O, L']
    qGp, sGp = orc.quant(GpT, 8, orc.SCALE_TENSOR)
    del GpT
    got = qgp_d.cpu().numpy()
    assert np.array_equal(sgp_d.cpu().numpy(), sGp)
    assert np.array_equal(got[:, :lp], qGp) and not got[:, lp:].any()
    # the g_x operands as in the paper-rule test; the products on sampled rows and columns
    qG, sG = orc.quant(orc.fwht_blocks_last(gyn, 16), 4, orc.SCALE_TENSOR)
    qW, sW = orc.quant(orc.fwht_blocks_first(wn, 16), 4, orc.SCALE_TENSOR)
    rng = np.random.default_rng(I)
    def sample(n):
        return np.unique(np.concatenate([[0, 255, 256, n - 1], rng.integers(0, n, 28)]))
    def deq(acc, sa, sb, div):
        return torch.from_numpy((((acc.astype(F32) * F32(sa)).astype(F32) * F32(sb)).astype(F32) / F32(div)).astype(F32)
                                ).to(torch.bfloat16)
    f32 = lambda a: a.astype(np.float32)
    f64 = lambda a: a.astype(np.float64)
    gx_c, gw_c = gx.cpu(), gw.cpu()
    r, c = sample(L), sample(I)
    assert torch.equal(gx_c[r], deq(f32(qG[r]) @ f32(qW), sG[0], sW[0], 16))
    assert torch.equal(gx_c[:, c], deq(f32(qG) @ f32(qW[:, c]), sG[0], sW[0], 16))
    r, c = sample(O), sample(I)
    assert torch.equal(gw_c[r], deq(np.rint(f64(qGp[r]) @ f64(xq_ref)), sGp[0], sx_ref[0], L))
    assert torch.equal(gw_c[:, c], deq(np.rint(f64(qGp) @ f64(xq_ref[:, c])), sGp[0], sx_ref[0], L))


def test_llama_layer_full_size_per_token_stochastic(gpu):
    """Llama-7B q/k/v/o (8192 tokens, 4096 -> 4096), bf16, Student-t gradient columns, with the quantisers
    the layer-wise selection picks most often: per-token steps and stochastic rounding on both g_y
    operands (norm_quantizer_BWD, utils/quant_matmul.py:19-31), n = 16 / r = 8.  Every code and step of
    both operands against the oracle under the same counter-based generator; the products on samples."""
    from hot_amd import ops
    L, O, I = 8192, 4096, 4096
    x, w, gy, heavy = llama_inputs(L, O, I, seed=99)
    ocfg = orc.HotConfig.paper(16, 8, gx_round=orc.ROUND_STOCH, gx_scale=orc.SCALE_ROW, gw_round=orc.ROUND_STOCH,
                               gw_scale=orc.SCALE_ROW, seed=21)
    opt = options_pair(ocfg)
    xd, wd, gyd = x.to(gpu), w.to(gpu), gy.to(gpu)
    xq, sx = ops.abc_forward(xd, opt)
    gx, gw = ops.linear_backward(gyd, wd, xq, sx, opt)
    qg_d, sg_d = ops.hq_rowwise(gyd, n=16, bits=4, rounding="stoch", scale="row", seed=21)
    qgp_d, sgp_d, lp = ops.hla_tokenwise(gyd, 16, list(ocfg.hla_rows), bits=8, rounding="stoch", scale="row", seed=21)
    torch.cuda.synchronize()
    gyn, wn, xn = gy.float().numpy(), w.float().numpy(), x.float().numpy()
    rows_sel = np.asarray(ocfg.hla_rows)
    xq_ref, sx_ref = orc.abc_forward(xn, ocfg)
    assert np.array_equal(xq.cpu().numpy()[:, :lp], xq_ref.T) and np.array_equal(sx.cpu().numpy(), sx_ref)
    qG, sG = orc.quant(orc.fwht_blocks_last(gyn, 16), 4, orc.SCALE_ROW, orc.ROUND_STOCH, seed=21, stream=orc.STREAM_GX)
    assert np.array_equal(sg_d.cpu().numpy(), sG)
    assert np.array_equal(orc.unpack_int4(qg_d.cpu().numpy())[:, :O], qG)
    GpT = np.ascontiguousarray(orc.fwht_blocks_first(gyn, 16, rows_sel).T)                   # [O, L']
    qGp, sGp = orc.quant(GpT, 8, orc.SCALE_ROW, orc.ROUND_STOCH, seed=21, stream=orc.STREAM_GW,
                         index=orc.colwise_rng_index(O, L // 16, rows_sel))
    del GpT
    assert np.array_equal(sgp_d.cpu().numpy(), sGp)
    assert np.array_equal(qgp_d.cpu().numpy()[:, :lp], qGp)
    qW, sW = orc.quant(orc.fwht_blocks_first(wn, 16), 4, orc.SCALE_TENSOR)
    rng = np.random.default_rng(3)
    def sample(n):
        return np.unique(np.concatenate([[0, 255, 256, n - 1], rng.integers(0, n, 28)]))
    def deq(acc, sa, sb, div):
        return torch.from_numpy((((acc.astype(F32) * sa.astype(F32)).astype(F32) * F32(sb)).astype(F32) / F32(div)).astype(F32)
                                ).to(torch.bfloat16)
    f32 = lambda a: a.astype(np.float32)
    f64 = lambda a: a.astype(np.float64)
    gx_c, gw_c = gx.cpu(), gw.cpu()
    r, c = sample(L), sample(I)
    assert torch.equal(gx_c[r], deq(f32(qG[r]) @ f32(qW), sG[r, None], sW[0], 16))
    assert torch.equal(gx_c[:, c], deq(f32(qG) @ f32(qW[:, c]), sG[:, None], sW[0], 16))
    r, c = sample(O), sample(I)
    assert torch.equal(gw_c[r], deq(np.rint(f64(qGp[r]) @ f64(xq_ref)), sGp[r, None], sx_ref[0], 16))
    assert torch.equal(gw_c[:, c], deq(np.rint(f64(qGp) @ f64(xq_ref[:, c])), sGp[:, None], sx_ref[0], 16))


# ------------------------------------------------------------ the whole ViT-B/16 step

def test_vit_b16_full_model_step(gpu):
    """ViT-B/16 (12 blocks, width 768, 12 heads, MLP 3072, 100 classes; random init), batch 128, bf16,
    every Linear / Conv2d swapped for the HOT layers, quantisers chosen per layer by the calibration
    pass: gradients finite, one dictionary entry pair per layer, and every parameter gradient pointing
    the way of the plain bf16 backward."""
    import torch.nn as nn
    from hot_amd import args, lqs
    from hot_amd import utils as hutils
    from hot_amd.quant_matmul import HQ_Conv2d, HQ_Linear
    from hot_amd.vit import ViT
    saved = {k: getattr(args, k) for k in dir(args) if not k.startswith("_") and not callable(getattr(args, k))}
    try:
        torch.manual_seed(0)
        model = ViT().to(gpu).to(torch.bfloat16)
        img = torch.randn(128, 3, 224, 224, device=gpu, dtype=torch.bfloat16)
        tgt = torch.randint(0, 100, (128,), device=gpu)
        args.plain_recipe()
        nn.functional.cross_entropy(model(img).float(), tgt).backward()
        plain = {n: p.grad.float().clone() for n, p in model.named_parameters()}
        model.zero_grad(set_to_none=True)
        hutils.replace_layers(model, nn.Conv2d, HQ_Conv2d)
        hutils.replace_layers(model, nn.Linear, HQ_Linear)
        hutils.name_layers(model)
        n_hot = sum(isinstance(m, (HQ_Linear, HQ_Conv2d)) for m in model.modules())
        assert n_hot == 1 + 12 * 4 + 1
        args.hot_recipe(gx="stoch", gw="stoch")
        args.batched_mode = "flatten"
        args.layer_quant_dict.clear()
        lqs.calibrate(model, [(img[:32], tgt[:32])], nn.CrossEntropyLoss())
        assert len(args.layer_quant_dict) == 2 * n_hot
        assert set(args.layer_quant_dict.values()) <= {"stoch_quantizer", "norm_quantizer"}
        args.quantAuto = True
        nn.functional.cross_entropy(model(img).float(), tgt).backward()
        torch.cuda.synchronize()
        worst = 1.0
        for n, p in model.named_parameters():
            assert p.grad is not None and bool(torch.isfinite(p.grad).all()), n
            if p.grad.numel() < 1024:
                continue
            cos = float(nn.functional.cosine_similarity(p.grad.float().flatten(), plain[n].flatten(), dim=0))
            worst = min(worst, cos)
            print("cosine %-32s %.3f" % (n, cos))
            # INT4 gradients through twelve blocks with a rank-reduced weight gradient: the direction is
            # kept, not the value
            assert cos > 0.4, (n, cos)
        assert worst < 0.9999            # the HOT path did run
    finally:
        for k, v in saved.items():
            setattr(args, k, v)
        args.layer_quant_dict.clear()
