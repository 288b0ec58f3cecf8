"""Host logic around the hot path: layer-wise quantizer selection, model surgery, precision
schedule, and the plain full-precision setting of the layers (all on CPU tensors)."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

from hot_amd import args, lqs
from hot_amd import utils as hutils
from hot_amd.quant_matmul import HQ_Conv2d, HQ_Linear, hot_switched_off, options_for
from hot_amd import ops


@pytest.fixture
def fresh_args():
    keys = [k for k in vars(args) if not k.startswith("_") and k not in ("defaultdict",)]
    saved = {k: copy.copy(getattr(args, k)) for k in keys}
    args.hot_recipe()          # the module defaults describe a plain layer, as the reference's do
    yield args
    for k, v in saved.items():
        setattr(args, k, v)


def test_stoch_quantizer_properties():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 48, generator=g) * 3e-3
    q, s = lqs.stoch_quantizer(x, 4, False, generator=g)
    assert float(s) == pytest.approx(float(x.abs().max()) / 7)
    y = x / (s + 1e-11)
    assert torch.equal(q, q.round()) and float(q.abs().max()) <= 7
    assert bool(((q >= torch.floor(y)) & (q <= torch.ceil(y))).all())      # a neighbour of the exact quotient
    # unbiased: the mean over many draws converges on the quotient (std of the mean <= 0.5 / sqrt(400))
    acc = torch.zeros_like(x)
    for _ in range(400):
        acc += lqs.stoch_quantizer(x, 4, False, generator=g)[0]
    assert float((acc / 400 - y).abs().max()) < 0.12
    # the largest element is hit exactly
    i = x.abs().argmax()
    assert abs(float(q.flatten()[i])) == 7


def test_stoch_quantizer_batched_has_one_step_per_sample():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 16, 8, generator=g) * torch.tensor([1.0, 10.0, 0.1]).view(3, 1, 1)
    q, s = lqs.stoch_quantizer(x, 8, True, generator=g)
    assert s.shape == (3,)
    assert torch.allclose(s, x.abs().flatten(1).amax(1) / 127)
    assert float((q * s.view(3, 1, 1) - x).abs().max()) <= float(s.max()) * 1.0001


def test_norm_quantizer_rows():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(32, 64, generator=g)
    x[5] *= 1e3
    xq, one = lqs.norm_quantizer(x, 4, False, generator=g)
    assert one == 1.0
    step = x.abs().amax(1, keepdim=True) / 7
    assert bool(((xq - x).abs() <= step * 1.0001).all())                    # within one step of ITS row
    codes = xq / step
    assert torch.allclose(codes, codes.round(), atol=1e-4)
    # 3-D input: rows of every sample
    x3 = torch.randn(2, 8, 16, generator=g)
    xq3, _ = lqs.norm_quantizer(x3, 4, True, generator=g)
    assert bool(((xq3 - x3).abs() <= x3.abs().amax(-1, keepdim=True) / 7 * 1.0001).all())


def test_quantisation_error_matches_bernoulli_variance():
    """E|x - Q(x)|^2 = s^2 * sum f (1 - f) for stochastic rounding with fractional parts f."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(256, 128, generator=g)
    s = x.abs().max() / 7
    f = (x.abs() / (s + 1e-11)) % 1.0
    expect = float(torch.sqrt((s * s * f * (1 - f)).sum()))
    got = lqs.quantisation_error(x, "stoch_quantizer", 4, generator=g)
    assert got == pytest.approx(expect, rel=0.03)


def test_selection_rule():
    g = torch.Generator().manual_seed(4)
    flat = torch.randn(128, 64, generator=g)
    assert lqs.select_for_layer(flat, generator=g) == ("stoch_quantizer", "stoch_quantizer")
    spiky = torch.randn(128, 64, generator=g)
    spiky[3, 5] = 1e4          # one outlier sets the tensor-wide step; per-token steps confine it to its row
    assert lqs.select_for_layer(spiky, generator=g) == ("norm_quantizer", "stoch_quantizer")
    # a mild spread improves the error, but by less than half: the per-tensor quantiser stays
    mild = torch.randn(128, 64, generator=g) * torch.linspace(0.8, 1.2, 128).view(-1, 1)
    e_s = lqs.quantisation_error(mild, "stoch_quantizer", generator=g)
    e_n = lqs.quantisation_error(mild, "norm_quantizer", generator=g)
    assert e_n < e_s and (e_s - e_n) < 0.5 * e_s
    assert lqs.select_for_layer(mild, generator=g) == ("stoch_quantizer", "stoch_quantizer")


class Tiny(nn.Module):
    def __init__(self):
        super().__init__()
        self.stem = nn.Conv2d(2, 16, kernel_size=2, stride=2)
        self.dw = nn.Conv2d(16, 16, kernel_size=3, padding=1, groups=16)
        self.block = nn.Sequential(nn.Linear(16, 32), nn.GELU(), nn.Linear(32, 16))
        self.head = nn.Linear(16, 4)

    def forward(self, x):
        x = self.dw(self.stem(x))                      # [B, 16, 4, 4]
        x = x.flatten(2).transpose(1, 2)               # [B, 16 tokens, 16]
        x = x + self.block(x)
        return self.head(x.mean(1))


def test_replace_layers_keeps_parameters(fresh_args):
    torch.manual_seed(0)
    m = Tiny()
    ptrs = {n: p.data_ptr() for n, p in m.named_parameters()}
    hutils.replace_layers(m, nn.Conv2d, HQ_Conv2d)
    hutils.replace_layers(m, nn.Linear, HQ_Linear)
    hutils.name_layers(m)
    assert isinstance(m.stem, HQ_Conv2d) and not isinstance(m.dw, HQ_Conv2d)          # depth-wise stays
    assert isinstance(m.block[0], HQ_Linear) and isinstance(m.block[2], HQ_Linear) and isinstance(m.head, HQ_Linear)
    assert {n: p.data_ptr() for n, p in m.named_parameters()} == ptrs
    assert m.block[2].layer_name == "block.2" and m.stem.layer_name == "stem"
    assert "hadamard_bs" not in m.state_dict() and "block.0.hadamard_out" not in m.state_dict()


def test_replace_layers_skips_lora_parts(fresh_args):
    class Lora(nn.Module):
        def __init__(self):
            super().__init__()
            self.base_layer = nn.Linear(8, 8)
            self.lora_A = nn.ModuleDict({"default": nn.Linear(8, 2)})
    m = Lora()
    args.HLQ_on_base, args.HLQ_on_decompose = False, False
    hutils.replace_layers(m, nn.Linear, HQ_Linear)
    assert not isinstance(m.base_layer, HQ_Linear) and not isinstance(m.lora_A["default"], HQ_Linear)
    args.HLQ_on_base, args.HLQ_on_decompose = True, True
    hutils.replace_layers(m, nn.Linear, HQ_Linear)
    assert isinstance(m.base_layer, HQ_Linear) and isinstance(m.lora_A["default"], HQ_Linear)


def test_precision_scheduler(fresh_args):
    args.quantBWDGogi, args.quantBWDWgt = "stoch", "sawb"
    hutils.precision_scheduler(0, max_bit=8, min_bit=4, milestones=[2, 5])
    assert (args.GogiQuantBit, args.weightQuantBit, args.GogwQuantBit, args.actQuantBit) == (8, 8, 8, 8)
    hutils.precision_scheduler(1, milestones=[2, 5])
    assert args.GogiQuantBit == 8
    hutils.precision_scheduler(2, milestones=[2, 5])
    assert (args.GogiQuantBit, args.weightQuantBit) == (4, 8)          # sawb weights keep their width
    hutils.precision_scheduler(5, milestones=[2, 5])
    assert args.GogiQuantBit == 4                                      # already at the floor


def test_plain_setting_equals_autograd(fresh_args):
    """Transforms off, quantisers "no": the layers are ordinary layers, forward and backward."""
    args.TransformGogi = args.TransformWgt = args.TransformGogw = args.TransformInput = False
    args.quantBWDGogi = args.quantBWDWgt = args.quantBWDGogw = args.quantBWDAct = "no"
    assert hot_switched_off()
    torch.manual_seed(0)
    ref = Tiny()
    hot = copy.deepcopy(ref)
    hutils.replace_layers(hot, nn.Conv2d, HQ_Conv2d)
    hutils.replace_layers(hot, nn.Linear, HQ_Linear)
    x = torch.randn(3, 2, 8, 8)
    y = torch.tensor([0, 3, 1])
    for m in (ref, hot):
        nn.functional.cross_entropy(m(x), y).backward()
    for (n1, p1), (n2, p2) in zip(ref.named_parameters(), hot.named_parameters()):
        assert n1 == n2 and torch.allclose(p1.grad, p2.grad, atol=1e-6, rtol=1e-5), n1


def test_partial_settings_raise(fresh_args):
    args.TransformGogi = False
    assert not hot_switched_off()
    with pytest.raises(NotImplementedError):
        options_for(128)


def test_calibrate_fills_dict_and_restores_args(fresh_args):
    torch.manual_seed(0)
    m = Tiny()
    hutils.replace_layers(m, nn.Conv2d, HQ_Conv2d)
    hutils.replace_layers(m, nn.Linear, HQ_Linear)
    hutils.name_layers(m)
    args.layer_quant_dict.clear()
    before = (args.TransformGogi, args.quantBWDGogi, args.quantAuto)
    batches = [(torch.randn(4, 2, 8, 8), torch.randint(0, 4, (4,))) for _ in range(2)]
    opt = torch.optim.AdamW(m.parameters(), lr=1e-3, eps=1e-11)
    out = lqs.calibrate(m, batches, nn.CrossEntropyLoss(), opt, generator=torch.Generator().manual_seed(0))
    assert (args.TransformGogi, args.quantBWDGogi, args.quantAuto) == before
    for layer in ("stem", "block.0", "block.2", "head"):
        assert out[layer + "_gx"] in lqs.quantScheme_gx and out[layer + "_gw"] == "stoch_quantizer"
    # the choice reaches the native options when quantAuto is on
    args.quantAuto = True
    out["block.0_gx"], out["block.0_gw"] = "norm_quantizer", "stoch_quantizer"
    o = options_for(128, "block.0")
    assert (o.gx_round, o.gx_scale, o.gw_round, o.gw_scale) == (ops.ROUND_STOCH, ops.SCALE_ROW, ops.ROUND_STOCH, ops.SCALE_TENSOR)
    assert o.gw_bits == args.GogiQuantBit       # the reference's g_W branch reads GogiQuantBit under quantAuto


def test_calibration_judges_the_first_batch(fresh_args):
    """The reference's tensor dictionary fills each slot once (utils/plot.py:175-177), so with several
    calibration batches the selection sees the gradients of the first one, taken before any weight
    update; keep="last" is the explicit alternative."""
    torch.manual_seed(1)
    m = nn.Sequential(nn.Linear(8, 8))
    hutils.replace_layers(m, nn.Linear, HQ_Linear)
    hutils.name_layers(m)
    args.plain_recipe()
    batches = [torch.randn(16, 8), 100.0 * torch.randn(16, 8)]
    seen = []
    for keep in ("first", "last"):
        cap = lqs.GradCapture(m, (HQ_Linear,), keep=keep)
        grads = []
        for b in batches:
            y = m(b.clone().requires_grad_(True))
            g = torch.randn_like(y)
            grads.append(g)
            y.backward(g)
        cap.close()
        (got,) = cap.grads.values()
        assert torch.equal(got, grads[0] if keep == "first" else grads[1])
        seen.append(got)
    assert not torch.equal(seen[0], seen[1])
    with pytest.raises(ValueError):
        lqs.GradCapture(m, (HQ_Linear,), keep="middle")


# ------------------------------------------------------------------ analytic calculators

def test_bops_formulas_by_hand():
    """utils/analysis_calculator.py:142-167 at a shape small enough to add up by hand."""
    from hot_amd.analysis_calculator import backward_bops, forward_bops
    L, O, I, r, n = 32, 8, 4, 8, 16
    assert forward_bops(L, O, I) == 32 * 8 * 4 * 1024
    assert backward_bops("FP", L, O, I) == backward_bops("LoRA", L, O, I) == 2 * 1024 * 1024
    assert backward_bops("LBP", L, O, I) == (256 * 4 + 128 * 4 + 32 * 32 * 0.5) * 1024
    assert backward_bops("LUQ", L, O, I) == 3 * (256 + 64 + 256) * 1024 + 2 * 1024 * 32
    gx = 256 * 4 + 32 * 4 + 256 + 32
    gw = 128 * 4 + 256 * 4 + 8 * 0.5 * 32 + 4 * 0.5 * 8
    assert backward_bops("HLQ", L, O, I) == (gx + gw + 32 + 128) * 1024 + 8 * 0.5 * 32 * 4 * 64 + 1024 * 16
    assert backward_bops("HLQ", L, O, I, frozen=True) == (gx + 128) * 1024 + 1024 * 16
    # HLQ replaces two fp32 products by an INT4 and a half-length INT8 one: far fewer bit operations at real sizes
    assert backward_bops("HLQ", 12608, 3072, 768) < 0.05 * backward_bops("FP", 12608, 3072, 768)
    with pytest.raises(NotImplementedError):
        backward_bops("other", 1, 1, 1)


def test_bops_counter_and_memory_calculator_on_a_small_model():
    from hot_amd.analysis_calculator import BOPsCounter, ModelMemoryCalculator, backward_bops, forward_bops
    torch.manual_seed(0)
    m = Tiny()
    c = BOPsCounter("HLQ")
    c.start_counting(m)
    m(torch.randn(2, 2, 8, 8))
    c.stop_counting()
    tot = c.get_total_gbops()
    # stem: 4 x 4 output positions, 16 out-channels, 2 * 2 * 2 in-features; block.0: [2, 16, 16] -> L = 16
    assert tot["forward_gbops_by_layer"]["stem"] == forward_bops(16, 16, 8)
    assert tot["backward_gbops_by_layer"]["block.0"] == backward_bops("HLQ", 16, 32, 16)
    assert tot["forward_gbops_by_layer"]["head"] == forward_bops(2, 4, 16)          # 2-D input: rows are the tokens
    assert tot["total_gbops"] == tot["total_forward_gbops"] + tot["total_backward_gbops"]
    c.reset()
    assert c.get_total_gbops()["total_gbops"] == 0

    params = sum(p.numel() for p in m.parameters())
    opt = torch.optim.AdamW(m.parameters())
    fp = ModelMemoryCalculator(m, (2, 8, 8), batch_size=4, optimizer=opt).get_total_memory()
    assert fp["parameters"] == fp["gradients"] == 4 * params and fp["optimizer_state"] == 8 * params
    # outputs of stem [16, 4, 4], dw [16, 4, 4], block.0 [16, 32], block.2 [16, 16], head [4] per sample
    outs = 256 + 256 + 512 + 256 + 4
    assert fp["activations"] == outs * 4 * 4
    hlq = ModelMemoryCalculator(m, (2, 8, 8), batch_size=4, optimizer=None, isHLQ=True).get_total_memory()
    assert hlq["activations"] == (128 + 128 + 256 + 128 + 2) * 4 and hlq["optimizer_state"] == 0
    m.head.weight.requires_grad_(False)
    frozen = ModelMemoryCalculator(m, (2, 8, 8), batch_size=4).get_total_memory()
    assert frozen["activations"] == (outs - 4) * 4 * 4 and frozen["parameters"] == 4 * (params - 64)
    assert ModelMemoryCalculator.format_bytes(3 * 1024 ** 3) == "3.00GB"
