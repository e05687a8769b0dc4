"""torch_ggml_ops for MI355X: matmul of bf16 activations with packed GGUF weights.

Importing the package loads the gfx950 library (C ABI in include/tgo.h) and registers the
six ``torch_ggml_ops::`` operators of the reference with their fake kernels and autograd formulas,
plus ``quantize_q8_1`` / ``mmq_prepared`` for several projections of one input and the
``*_gathered`` grouped operators that fold the token -> sorted-row gather into the quantizer,
the routing sort / weighted combine of a mixture-of-experts layer (``route``, ``moe_combine``,
``grouped_mmq_combine``, ``moe_layer``),
``grouped_mmq_swiglu``, the gate/up pair with the activation fused into the kernel's epilogue, and
``chunked_lm_head_loss``, the cross-entropy through a packed LM head one chunk of rows at a time.
"""

import torch  # noqa: F401  (operators are registered against the loaded torch)

from . import _native  # noqa: F401  loads libtgo_hip.so or fails loudly
from .gathered import grouped_mmq_gathered, grouped_mmq_pair_gathered
from .grouped_mmq import grouped_mmq, grouped_mmq_pair
from .lm_head import chunked_lm_head_loss
from .mmq import mmq
from .moe import grouped_mmq_combine, moe_combine, moe_layer, route
from .prepared import mmq_multi, mmq_prepared, quantize_q8_1
from .swiglu import grouped_mmq_swiglu

__all__ = [
    "chunked_lm_head_loss",
    "grouped_mmq",
    "grouped_mmq_combine",
    "grouped_mmq_gathered",
    "grouped_mmq_pair",
    "grouped_mmq_pair_gathered",
    "grouped_mmq_swiglu",
    "mmq",
    "mmq_multi",
    "mmq_prepared",
    "moe_combine",
    "moe_layer",
    "quantize_q8_1",
    "route",
]
