"""Gate/up pair with the SwiGLU activation applied in the kernel's epilogue.

``grouped_mmq_pair`` returns the gate and up projections and the caller computes
``silu(gate) * up`` (two more passes over ``2 x rows x out_features`` bf16).  Here a workgroup runs
the gate tile, then the up tile of the same rows and columns, and stores ``silu(gate) * up``
directly: the up projection never reaches memory and no activation kernel runs.  Both factors are
rounded to bf16 first, as the caller-side computation would see them, and the product is rounded
once.  The reference has no such operator (its pair operator ends at the two projections,
csrc/mmq_hip.cu:1054-1193).

The gradient with respect to the input recomputes the up projection (one grouped forward) instead
of keeping it -- except for calls large enough for the scaled operands, whose kernel writes the up
projection anyway: the operator then keeps it (its third, internal output).  The gate is saved, ``d_gate`` and ``d_up`` follow from one elementwise kernel
(``tgo_swiglu_backward``), and the fused pair grad-input finishes.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import _native
from .grouped_mmq import _forward as _grouped_forward
from .gathered import _rows_grad_input, _scatter_to_tokens

torch.library.define(
    "torch_ggml_ops::grouped_mmq_swiglu",
    "(Tensor input, Tensor? row_index, Tensor gate_packed_weight, Tensor up_packed_weight, Tensor expert_indices, "
    "Tensor expert_offsets, int quant_type, int out_features) -> (Tensor, Tensor, Tensor)",
)


def _keeps_up(quant_type: int, rows: int, out_features: int) -> bool:
    """Calls large enough for the scaled operands write the up projection anyway (their kernel has no fused epilogue);
    the operator then keeps it for the backward pass instead of computing it a second time there."""
    return _native.forward_operand_for(int(quant_type), int(rows), int(out_features), 2) == "scaled"


@torch.library.impl("torch_ggml_ops::grouped_mmq_swiglu", "CUDA")
def _swiglu_device(
    input, row_index, gate_packed_weight, up_packed_weight, expert_indices, expert_offsets, quant_type, out_features
):
    rows = input.shape[0] if row_index is None else row_index.shape[0]
    if _keeps_up(quant_type, rows, out_features):
        # what tgo_grouped_mmq_swiglu does for such a call, with the activation written beside the up projection
        # instead of over it
        gate, up = _grouped_forward(
            input, gate_packed_weight, up_packed_weight, expert_indices, expert_offsets, quant_type, out_features, row_index
        )
        activated = torch.empty_like(up)
        with _native.on_device(gate.device):
            _native.check(
                _native.lib.tgo_swiglu_rows(
                    gate.data_ptr(), up.data_ptr(), activated.data_ptr(), gate.numel(),
                    _native.stream_of(gate.device),
                )
            )
        return activated, gate, up
    gate, activated = _grouped_forward(
        input, gate_packed_weight, up_packed_weight, expert_indices, expert_offsets, quant_type, out_features,
        row_index, swiglu=True,
    )
    return activated, gate, input.new_empty((0, out_features))


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_swiglu")
def _swiglu_fake(
    input, row_index, gate_packed_weight, up_packed_weight, expert_indices, expert_offsets, quant_type, out_features
):
    rows = input.shape[0] if row_index is None else row_index.shape[0]
    kept = rows if _keeps_up(quant_type, rows, out_features) else 0
    return (
        input.new_empty((rows, out_features)), input.new_empty((rows, out_features)), input.new_empty((kept, out_features))
    )


def _activation_backward(gate, up, grad_activated, grad_gate):
    """(d_gate, d_up) of ``silu(gate) * up`` for the cotangent ``grad_activated`` (plus ``grad_gate``, a cotangent of
    the gate output itself, or None): one elementwise kernel, bf16 in and out, fp32 arithmetic."""
    tensors = [gate, up, grad_activated] + ([] if grad_gate is None else [grad_gate])
    gate, up, grad_activated, *rest = [t.contiguous() for t in tensors]
    d_gate, d_up = torch.empty_like(gate), torch.empty_like(gate)
    with _native.on_device(gate.device):
        _native.check(
            _native.lib.tgo_swiglu_backward(
                gate.data_ptr(), up.data_ptr(), grad_activated.data_ptr(), rest[0].data_ptr() if rest else None,
                d_gate.data_ptr(), d_up.data_ptr(), gate.numel(), _native.stream_of(gate.device),
            )
        )
    return d_gate, d_up


def _setup_context(ctx, inputs, output) -> None:
    input, row_index, gate_weight, up_weight, expert_indices, expert_offsets, quant_type, out_features = inputs
    ctx.quant_type, ctx.out_features = quant_type, out_features
    ctx.tokens, ctx.in_features = input.shape
    ctx.gathered = row_index is not None
    if ctx.needs_input_grad[0]:
        ctx.save_for_backward(
            input, row_index, gate_weight, up_weight, expert_indices, expert_offsets, output[1], output[2]
        )


def _backward(ctx, grad_activated, grad_gate, grad_up):
    grad_input = None
    if ctx.needs_input_grad[0] and (grad_activated is not None or grad_gate is not None or grad_up is not None):
        input, row_index, gate_weight, up_weight, expert_indices, expert_offsets, gate, up = ctx.saved_tensors
        d_gate = grad_gate
        d_up = grad_up if up.shape[0] > 0 else None   # (the third output is a placeholder when the up projection is not kept)
        if grad_activated is not None:
            if up.shape[0] == 0:
                up = _grouped_forward(
                    input, up_weight, None, expert_indices, expert_offsets, ctx.quant_type, ctx.out_features, row_index
                )[0]
            d_gate, through_up = _activation_backward(gate, up, grad_activated, grad_gate)
            d_up = through_up if d_up is None else d_up + through_up
        if d_gate is None:
            d_gate = torch.zeros_like(gate)
        if d_up is not None:
            grad_rows = _rows_grad_input(
                d_gate, d_up, gate_weight, up_weight, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
            )
        else:
            grad_rows = _rows_grad_input(
                d_gate, None, gate_weight, None, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
            )
        grad_input = _scatter_to_tokens(grad_rows, row_index, ctx.tokens) if ctx.gathered else grad_rows
    return grad_input, None, None, None, None, None, None, None


torch.library.register_autograd("torch_ggml_ops::grouped_mmq_swiglu", _backward, setup_context=_setup_context)


def grouped_mmq_swiglu(
    input: torch.Tensor,
    gate_packed_weight: torch.Tensor,
    up_packed_weight: torch.Tensor,
    expert_indices: torch.Tensor,
    expert_offsets: torch.Tensor,
    quant_type: int,
    out_features: int,
    row_index: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``silu(gate) * up`` of the grouped gate/up pair, ``[rows, out_features]`` bf16.

    ``input`` holds expert-sorted rows, or token rows when ``row_index`` (the token of each sorted row) is given.
    Rows that no valid group covers are left uninitialised, as for ``grouped_mmq``.
    """
    activated, _gate, _up = torch.ops.torch_ggml_ops.grouped_mmq_swiglu.default(
        input, row_index, gate_packed_weight, up_packed_weight, expert_indices, expert_offsets,
        int(quant_type), int(out_features),
    )
    return activated


__all__ = ["grouped_mmq_swiglu"]
