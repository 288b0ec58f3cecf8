"""Analytic cost models of the reference (utils/analysis_calculator.py): bit operations of a
training step per layer and the memory footprint of a model.  Host-side arithmetic on shapes only;
nothing here touches the kernels.

Bit operations (BOPsCounter, utils/analysis_calculator.py:135-240): a multiply-accumulate of an a-bit
by a b-bit operand counts a*b bit operations; element-wise fp32 work counts 32*32 per element.
With L tokens, O out-features, I in-features, Hadamard block n and kept rows r:

  forward            L O I 32^2
  FP / LoRA backward 2 L O I 32^2                                  (two fp32 products)
  LBP                (L O log2 n + L I log2 n + O I L r/n) 32^2
  LUQ                3 (L O + 2 O I + 2 L I) 32^2 + 2 (L O I 4*4*2)
  HLQ                (L O log2 n + O I log2 n + L O + O I          g_x path: transforms, quantisers
                      + L I log2 n + L O log2 n + O L r/n + I O r/n   g_W path (absent in a frozen layer)
                      + I O + L I) 32^2                            dequantisation
                     + O (r/n) L I 8*8 + L O I 4*4                 the INT8 and INT4 products
(a frozen "base_layer" of a LoRA model has no weight gradient: its HLQ cost keeps the g_x path, the L I
dequantisation and the INT4 product only, :155-159).  The reference fixes n = 16, r = 8 (:176-177, :193-194).
"""
from __future__ import annotations

import math
from collections import defaultdict
from typing import Any, Dict, Optional, Tuple

import torch
import torch.nn as nn

FP_BITS = 32 * 32
SCHEMES = ("FP", "LoRA", "LBP", "LUQ", "HLQ")


def backward_bops(scheme: str, L: int, O: int, I: int, r: int = 8, n: int = 16, frozen: bool = False) -> float:
    """Bit operations of one layer's backward under `scheme` (utils/analysis_calculator.py:142-167)."""
    lg = math.log2(n)
    if scheme in ("FP", "LoRA"):
        return 2.0 * L * O * I * FP_BITS
    if scheme == "LBP":
        return (L * O * lg + L * I * lg + O * I * L * (r / n)) * FP_BITS
    if scheme == "LUQ":
        return 3.0 * (L * O + 2 * O * I + 2 * L * I) * FP_BITS + 2.0 * L * O * I * (4 * 4 * 2)
    if scheme == "HLQ":
        gx_path = L * O * lg + O * I * lg + L * O + O * I
        if frozen:
            return (gx_path + L * I) * FP_BITS + L * O * I * (4 * 4)
        gw_path = L * I * lg + L * O * lg + O * (r / n) * L + I * (r / n) * O
        return (gx_path + gw_path + I * O + L * I) * FP_BITS + O * (r / n) * L * I * (8 * 8) + L * O * I * (4 * 4)
    raise NotImplementedError("scheme %r (one of %s)" % (scheme, ", ".join(SCHEMES)))


def forward_bops(L: int, O: int, I: int) -> float:
    return float(L) * O * I * FP_BITS


class BOPsCounter:
    """Forward hooks on every Conv2d / Linear that record the layer's forward and backward bit
    operations for one sample (tokens = the second dimension of a 3-D input, else the first; output
    positions for a convolution, whose in-features are C k k)."""

    def __init__(self, transform_scheme: str, r: int = 8, n: int = 16):
        if transform_scheme not in SCHEMES:
            raise NotImplementedError("scheme %r (one of %s)" % (transform_scheme, ", ".join(SCHEMES)))
        self.transform_scheme = transform_scheme
        self.r, self.n = r, n
        self.forward_gbops: Dict[str, float] = defaultdict(int)
        self.backward_gbops: Dict[str, float] = defaultdict(int)
        self.handles = []

    def layer_shape(self, module: nn.Module, input_shape, output_shape) -> Tuple[int, int, int]:
        if isinstance(module, nn.Conv2d):
            L = int(output_shape[-1]) * int(output_shape[-2])
            return L, module.out_channels, module.kernel_size[0] * module.kernel_size[1] * module.in_channels
        L = int(input_shape[1]) if len(input_shape) == 3 else int(input_shape[0])
        return L, module.out_features, module.in_features

    def hook_fn(self, name: str):
        def hook(module, inputs, output):
            L, O, I = self.layer_shape(module, inputs[0].shape, output.shape)
            self.forward_gbops[name] = forward_bops(L, O, I)
            self.backward_gbops[name] = backward_bops(self.transform_scheme, L, O, I, self.r, self.n,
                                                      frozen="base_layer" in name)
        return hook

    def start_counting(self, model: nn.Module) -> None:
        for name, module in model.named_modules():
            if isinstance(module, (nn.Conv2d, nn.Linear)):
                self.handles.append(module.register_forward_hook(self.hook_fn(name)))

    def stop_counting(self) -> None:
        for h in self.handles:
            h.remove()
        self.handles = []

    def get_total_gbops(self) -> Dict[str, Any]:
        fwd, bwd = sum(self.forward_gbops.values()), sum(self.backward_gbops.values())
        return {"total_forward_gbops": fwd, "total_backward_gbops": bwd, "total_gbops": fwd + bwd,
                "forward_gbops_by_layer": dict(self.forward_gbops), "backward_gbops_by_layer": dict(self.backward_gbops)}

    def reset(self) -> None:
        self.forward_gbops.clear()
        self.backward_gbops.clear()


class ModelMemoryCalculator:
    """Bytes of a training step (utils/analysis_calculator.py:11-133): parameters and gradients of the
    trainable tensors (a fused "qkv" tensor counted three times, :37-40), the activations saved by every
    trainable Conv2d / Linear (one dummy sample through the model, scaled by the batch; with isHLQ half a
    byte per output element, i.e. the INT8 buffer at 50 % kept rows, :53-57; "qkv" layers four times), and
    two AdamW moments per parameter."""

    def __init__(self, model: nn.Module, input_size: Tuple, batch_size: int,
                 optimizer: Optional[torch.optim.Optimizer] = None, isHLQ: bool = False, run_name: str = "",
                 dtype: torch.dtype = torch.float32):
        self.model, self.input_size, self.batch_size = model, tuple(input_size), int(batch_size)
        self.optimizer, self.isHLQ, self.run_name = optimizer, bool(isHLQ), run_name
        self.bytes_per_element = torch.finfo(dtype).bits // 8

    def get_parameter_memory(self) -> Dict[str, float]:
        out: Dict[str, float] = {}
        total = 0
        for name, p in self.model.named_parameters():
            if not p.requires_grad:
                continue
            count = p.numel() * (3 if "qkv" in name else 1)
            out[name] = count * self.bytes_per_element
            total += count
        out["total"] = total * self.bytes_per_element
        return out

    def get_activation_memory(self) -> Dict[str, float]:
        sizes: Dict[str, float] = {}

        def hook_fn(name):
            def hook(module, inputs, output):
                if not module.weight.requires_grad:
                    sizes[name] = 0
                elif self.isHLQ:
                    sizes[name] = (output.numel() // 2) * self.batch_size
                else:
                    sizes[name] = output.numel() * self.batch_size * self.bytes_per_element
                if "qkv" in name:
                    sizes[name] *= 4
            return hook

        hooks = [m.register_forward_hook(hook_fn(n)) for n, m in self.model.named_modules()
                 if isinstance(m, (nn.Conv2d, nn.Linear))]
        try:
            first = next(self.model.parameters(), None)
            device = first.device if first is not None else torch.device("cpu")
            dt = first.dtype if first is not None and first.dtype.is_floating_point else torch.float32
            with torch.no_grad():
                self.model(torch.randn(1, *self.input_size, device=device, dtype=dt))
        finally:
            for h in hooks:
                h.remove()
        return sizes

    def get_gradient_memory(self) -> float:
        return self.get_parameter_memory()["total"]

    def get_optimizer_state_memory(self) -> Dict[str, float]:
        if isinstance(self.optimizer, torch.optim.AdamW):
            return {"total": 2 * self.get_parameter_memory()["total"]}
        return {"total": 0}

    def get_total_memory(self) -> Dict[str, float]:
        params = self.get_parameter_memory()["total"]
        acts = sum(self.get_activation_memory().values())
        grads = self.get_gradient_memory()
        opt = self.get_optimizer_state_memory()["total"]
        return {"parameters": params, "activations": acts, "gradients": grads, "optimizer_state": opt,
                "total": params + acts + grads + opt}

    @staticmethod
    def format_bytes(nbytes: float) -> str:
        return "%.2fGB" % (nbytes / 1024 ** 3)

    def print_memory_usage(self) -> None:
        m = self.get_total_memory()
        print("===== Analysis of Memory footprint: %s-%d=====" % (self.run_name, self.batch_size))
        for label, key in (("Weight", "parameters"), ("Activation", "activations"), ("Gradient", "gradients"),
                           ("Optimizer State", "optimizer_state"), ("Total", "total")):
            print("%s: %s" % (label, self.format_bytes(m[key])))
        print("=========================================")
