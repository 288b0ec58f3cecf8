"""Module-global options, with the names the reference's hot path reads from
its own ``args`` module (args.py:29-49; defaults of ViT_main.py:94-113 and the
canonical recipe of main.sh:14-24).

`hot_amd.quant_matmul` reads these on every call, exactly as the reference's
FLinearQ does, so code that mutates ``args.<flag>`` keeps working.  Only the
scheme ``gih_gwlr`` with all four transforms on is implemented natively.
"""
from collections import defaultdict

BATCH_SIZE = 0

GogiQuantBit = 4     # g_y . H          (g_x path, A operand)
weightQuantBit = 4   # H . W            (g_x path, B operand)
GogwQuantBit = 8     # (P g_y)^T        (g_W path, A operand)
actQuantBit = 8      # P x              (g_W path, B operand; the saved buffer)

eps = 1e-11

precisionScheduling = False   # utils.precision_scheduler drives the bit widths per epoch
milestone = " "

quantAuto = False
quantBWDGogi = "int"   # int | stoch | nq      ("no" on all four + Transform* off = plain layer)
quantBWDWgt = "int"    # int | stoch | sawb
quantBWDGogw = "int"   # int | stoch | nq
quantBWDAct = "int"    # int | stoch | sawb

vectorPercentile = 50

transform_scheme = "gih_gwlr"
TransformGogi = True
TransformWgt = True
TransformGogw = True
TransformInput = True

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
