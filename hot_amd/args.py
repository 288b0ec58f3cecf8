"""Module-global options, with the names the reference's hot path reads from
its own ``args`` module (args.py:29-49; defaults of ViT_main.py:94-113 and the
canonical recipe of main.sh:14-24).

`hot_amd.quant_matmul` reads these on every call, exactly as the reference's
FLinearQ does, so code that mutates ``args.<flag>`` keeps working.  The
defaults are the reference's own (args.py:29-49): every transform off, every
quantiser "no", widths 0 -- a plain full-precision layer, until a trainer (or
one of the recipes below) sets the flags.
"""
from collections import defaultdict

BATCH_SIZE = 0

GogiQuantBit = 0     # g_y . H          (g_x path, A operand)
weightQuantBit = 0   # H . W            (g_x path, B operand)
GogwQuantBit = 0     # (P g_y)^T        (g_W path, A operand)
actQuantBit = 0      # P x              (g_W path, B operand; the saved buffer)

eps = 1e-11

precisionScheduling = False   # utils.precision_scheduler drives the bit widths per epoch
milestone = " "

quantAuto = False
quantBWDGogi = "no"    # int | stoch | nq | luq   ("no" on all four + Transform* off = plain layer)
quantBWDWgt = "no"     # int | stoch | sawb
quantBWDGogw = "no"    # int | stoch | nq | luq
quantBWDAct = "no"     # int | stoch | sawb

vectorPercentile = 50

transform_scheme = "gih_gwlr"
TransformGogi = False
TransformWgt = False
TransformGogw = False
TransformInput = False

HLQ_on_base = False
HLQ_on_decompose = False

layer_quant_dict = defaultdict()

# ---- options without a counterpart in the reference -------------------------
# Token-dimension rule for the low-rank projection: "python" = the reference's
# make_WHT rule on the token count, "paper" = n 16 / 8 lowest sequencies.
hla_rule = "python"
# Largest token block of the python rule.  The reference takes the largest power of two dividing the
# token count, whatever it is (8192 tokens -> n = 8192, r = 2080); blocks up to 64 tokens run in the
# fast one-pass kernels, larger ones in an exact two-level path through an fp32 workspace.  Lower this
# (for example to 64: then n = 64, r = 36) to trade the reference's compression ratio for speed.
hla_max_block = 8192
# 3-D activations [B, L, C]: "per_sample" follows the reference (one call and one
# set of steps per sample), "flatten" treats them as [B*L, C].
batched_mode = "per_sample"
# Key of the counter-based generator used for stochastic rounding; the step
# counter below is added to it and advanced after every backward call.
sr_seed = 0
sr_step = 0


# ---- recipes ------------------------------------------------------------------
def _set(**kw) -> None:
    g = globals()
    for k, v in kw.items():
        g[k] = v


def hot_recipe(gx_bits: int = 4, w_bits: int = 4, gw_bits: int = 8, act_bits: int = 8, gx: str = "int",
               w: str = "int", gw: str = "int", act: str = "int", scheme: str = "gih_gwlr", auto: bool = False) -> None:
    """Switches the HOT path on: all four transforms, the given quantisers and widths.  The defaults
    are the deterministic setting (round-to-nearest absmax quantisers, INT4 g_x path, INT8 g_W path)."""
    _set(transform_scheme=scheme, TransformGogi=True, TransformWgt=True, TransformGogw=True, TransformInput=True,
         GogiQuantBit=gx_bits, weightQuantBit=w_bits, GogwQuantBit=gw_bits, actQuantBit=act_bits,
         quantBWDGogi=gx, quantBWDWgt=w, quantBWDGogw=gw, quantBWDAct=act, quantAuto=auto)


def canonical_recipe() -> None:
    """The reference's training recipe: main.sh:14-24 (scheme gih_gwlr, all transforms, widths 4/4/8/8)
    over the trainer's defaults ViT_main.py:100-106 (quantAuto on, per-token stochastic g_y quantisers
    unless the layer-wise selection says otherwise, SAWB for weights and activations)."""
    hot_recipe(4, 4, 8, 8, gx="nq", w="sawb", gw="nq", act="sawb", auto=True)


def plain_recipe() -> None:
    """Back to the reference's module defaults: a full-precision layer."""
    _set(TransformGogi=False, TransformWgt=False, TransformGogw=False, TransformInput=False,
         GogiQuantBit=0, weightQuantBit=0, GogwQuantBit=0, actQuantBit=0,
         quantBWDGogi="no", quantBWDWgt="no", quantBWDGogw="no", quantBWDAct="no", quantAuto=False)
