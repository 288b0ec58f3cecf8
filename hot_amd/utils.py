"""Model surgery and the precision schedule of the reference's utils/utils.py
(:53-74 replace_layers, :149-159 precision_scheduler), for models built from
``hot_amd.quant_matmul`` layers."""
from __future__ import annotations

import torch.nn as nn

from . import args


def _adopt(parent: nn.Module, child_name: str, new_layer: nn.Module, old_layer: nn.Module) -> None:
    # the new layer takes over the parameters themselves (no copy), like the reference
    new_layer.weight.data = old_layer.weight.data
    new_layer.weight.requires_grad = old_layer.weight.requires_grad
    if old_layer.bias is not None:
        new_layer.bias.data = old_layer.bias.data
    setattr(parent, child_name, new_layer)


def replace_layers(model: nn.Module, old, new) -> None:
    """Swaps every ``old`` layer (nn.Linear or nn.Conv2d) below `model` for ``new`` in place.

    Grouped (depth-wise) convolutions stay as they are; LoRA's ``base_layer`` / ``default`` linears
    are only replaced when ``args.HLQ_on_base`` / ``args.HLQ_on_decompose`` say so."""
    for name, module in list(model.named_children()):
        if len(list(module.children())) > 0:
            replace_layers(module, old, new)
        if old is nn.Conv2d and isinstance(module, nn.Conv2d) and module.groups == 1:
            layer = new(module.in_channels, module.out_channels, kernel_size=module.kernel_size,
                        stride=module.stride, padding=module.padding)
            _adopt(model, name, layer, module)
        elif old is nn.Linear and isinstance(module, nn.Linear):
            if "base_layer" in name and not args.HLQ_on_base:
                continue
            if "default" in name and not args.HLQ_on_decompose:
                continue
            layer = new(module.in_features, module.out_features)
            _adopt(model, name, layer, module)


def name_layers(model: nn.Module) -> None:
    """Gives every HOT layer its module path as ``layer_name`` (ViT_main.py:158-160): the key under
    which the layer-wise quantizer selection stores its choice."""
    from .quant_matmul import HQ_Conv2d, HQ_Linear
    for name, layer in model.named_modules():
        if isinstance(layer, (HQ_Linear, HQ_Conv2d)):
            layer.layer_name = name


def precision_scheduler(current_epoch, max_bit=8, min_bit=4, milestones=()):
    """Starts every operand at `max_bit`; at each milestone epoch halves the bit width of the g_x
    product's operands (g_y . H and H . W) while every width is still above `min_bit`."""
    if current_epoch == 0:
        args.GogiQuantBit = args.weightQuantBit = args.GogwQuantBit = args.actQuantBit = max_bit
    elif current_epoch in milestones and min(args.GogiQuantBit, args.weightQuantBit, args.GogwQuantBit,
                                             args.actQuantBit) > min_bit:
        if args.quantBWDGogi in ("stoch", "int"):
            args.GogiQuantBit = args.GogiQuantBit // 2
        if args.quantBWDWgt in ("stoch", "int"):
            args.weightQuantBit = args.weightQuantBit // 2
