"""Grouped operators that take unsorted token activations plus the sorted-row gather index.

A mixture-of-experts layer routes ``tokens`` activations to ``rows = tokens * top_k`` expert-sorted
rows.  The reference's grouped operators want those rows materialised
(``hidden.index_select(0, row_index)``, torch_ggml_ops/grouped_mmq.py:216 takes pre-sorted rows),
which reads and writes ``rows x in_features`` bf16 before the quantizer reads them again.  Here the
quantizer reads row ``row_index[r]`` of the token activations directly, so the sorted copy never
exists; results are bit-identical to ``grouped_mmq(hidden.index_select(0, row_index), ...)``.

The gradient with respect to the token activations is the grouped grad-input of the sorted rows
summed back per token in fp32 and rounded once.  An entry of ``row_index`` outside ``[0, tokens)``
(for example -1 for a dropped token) reads as a row of zeros in the forward and receives no
gradient in the backward.
"""

from __future__ import annotations

import torch

from . import _native
from .grouped_mmq import _forward as _grouped_forward
from .grouped_mmq import _grad_input as _grouped_grad_input

torch.library.define(
    "torch_ggml_ops::grouped_mmq_gathered",
    "(Tensor input, Tensor row_index, Tensor packed_weight, Tensor expert_indices, Tensor expert_offsets, "
    "int quant_type, int out_features) -> Tensor",
)
torch.library.define(
    "torch_ggml_ops::grouped_mmq_pair_gathered",
    "(Tensor input, Tensor row_index, Tensor first_packed_weight, Tensor second_packed_weight, "
    "Tensor expert_indices, Tensor expert_offsets, int quant_type, int out_features) -> (Tensor, Tensor)",
)


@torch.library.impl("torch_ggml_ops::grouped_mmq_gathered", "CUDA")
def _gathered_device(input, row_index, packed_weight, expert_indices, expert_offsets, quant_type, out_features):
    return _grouped_forward(
        input, packed_weight, None, expert_indices, expert_offsets, quant_type, out_features, row_index
    )[0]


@torch.library.impl("torch_ggml_ops::grouped_mmq_pair_gathered", "CUDA")
def _pair_gathered_device(
    input, row_index, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
):
    return _grouped_forward(
        input, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features,
        row_index,
    )


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_gathered")
def _gathered_fake(input, row_index, packed_weight, expert_indices, expert_offsets, quant_type, out_features):
    return input.new_empty((row_index.shape[0], out_features))


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_pair_gathered")
def _pair_gathered_fake(
    input, row_index, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
):
    shape = (row_index.shape[0], out_features)
    return input.new_empty(shape), input.new_empty(shape)


def _rows_grad_input(first_grad, second_grad, first_weight, second_weight, expert_indices, expert_offsets, quant_type, in_features):
    """Grouped grad-input of the sorted rows with uncovered rows cleared, so that they add nothing per token."""
    return _grouped_grad_input(
        first_grad.contiguous(), None if second_grad is None else second_grad.contiguous(), first_weight, second_weight,
        expert_indices, expert_offsets, quant_type, in_features, zero_fill=True,
    )


def _token_runs(row_index: torch.Tensor, tokens: int):
    """The sorted rows listed token by token: ``order[starts[t]:starts[t + 1]]`` are the rows of token ``t`` in row
    order.  Rows whose index names no token sort behind the last run (``starts[tokens]`` ends before them)."""
    present = (row_index >= 0) & (row_index < tokens)
    key = torch.where(present, row_index, tokens)
    sorted_key, order = torch.sort(key, stable=True)
    starts = torch.searchsorted(sorted_key, torch.arange(tokens + 1, device=key.device, dtype=key.dtype))
    return order, starts


def _scatter_to_tokens(grad_rows: torch.Tensor, row_index: torch.Tensor, tokens: int) -> torch.Tensor:
    """Sum of the sorted rows' gradients per token: fp32 accumulation in row order, one rounding to bf16.

    Rows whose index lies outside ``[0, tokens)`` were zeros in the forward and are dropped here.  The rows are
    listed token by token with a stable sort of the index (absent rows sort behind the last token), and one kernel
    adds each token's rows in that order (``tgo_rows_to_tokens``): no atomics, so the result does not depend on
    scheduling, and no data-dependent shapes, so the backward can be captured in a graph.
    """
    grad_rows = grad_rows.contiguous()
    order, starts = _token_runs(row_index, tokens)
    out = torch.empty((tokens, grad_rows.shape[1]), dtype=grad_rows.dtype, device=grad_rows.device)
    with _native.on_device(grad_rows.device):
        _native.check(
            _native.lib.tgo_rows_to_tokens(
                grad_rows.data_ptr(), order.data_ptr(), starts.data_ptr(), out.data_ptr(), tokens, grad_rows.shape[0],
                grad_rows.shape[1], _native.stream_of(grad_rows.device),
            )
        )
    return out


def _setup_gathered_context(ctx, inputs, output) -> None:
    input, row_index, packed_weight, expert_indices, expert_offsets, quant_type, _out_features = inputs
    ctx.quant_type = quant_type
    ctx.tokens, ctx.in_features = input.shape
    if ctx.needs_input_grad[0]:
        ctx.save_for_backward(row_index, packed_weight, expert_indices, expert_offsets)


def _gathered_backward(ctx, grad_output):
    grad_input = None
    if ctx.needs_input_grad[0]:
        row_index, packed_weight, expert_indices, expert_offsets = ctx.saved_tensors
        grad_rows = _rows_grad_input(
            grad_output, None, packed_weight, None, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
        )
        grad_input = _scatter_to_tokens(grad_rows, row_index, ctx.tokens)
    return grad_input, None, None, None, None, None, None


torch.library.register_autograd(
    "torch_ggml_ops::grouped_mmq_gathered", _gathered_backward, setup_context=_setup_gathered_context
)


def _setup_pair_gathered_context(ctx, inputs, output) -> None:
    input, row_index, first_weight, second_weight, expert_indices, expert_offsets, quant_type, _out_features = inputs
    ctx.quant_type = quant_type
    ctx.tokens, ctx.in_features = input.shape
    if ctx.needs_input_grad[0]:
        ctx.save_for_backward(row_index, first_weight, second_weight, expert_indices, expert_offsets)


def _pair_gathered_backward(ctx, first_grad_output, second_grad_output):
    grad_input = None
    if ctx.needs_input_grad[0]:
        row_index, first_weight, second_weight, expert_indices, expert_offsets = ctx.saved_tensors
        grad_rows = None
        if first_grad_output is not None and second_grad_output is not None:
            grad_rows = _rows_grad_input(
                first_grad_output, second_grad_output, first_weight, second_weight,
                expert_indices, expert_offsets, ctx.quant_type, ctx.in_features,
            )
        elif first_grad_output is not None:
            grad_rows = _rows_grad_input(
                first_grad_output, None, first_weight, None, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
            )
        elif second_grad_output is not None:
            grad_rows = _rows_grad_input(
                second_grad_output, None, second_weight, None, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
            )
        if grad_rows is not None:
            grad_input = _scatter_to_tokens(grad_rows, row_index, ctx.tokens)
    return grad_input, None, None, None, None, None, None, None


torch.library.register_autograd(
    "torch_ggml_ops::grouped_mmq_pair_gathered", _pair_gathered_backward, setup_context=_setup_pair_gathered_context
)


def grouped_mmq_gathered(
    input, row_index, packed_weight, expert_indices, expert_offsets, quant_type, out_features
) -> torch.Tensor:
    """``grouped_mmq(input.index_select(0, row_index), ...)`` without the sorted copy of the activations."""
    return torch.ops.torch_ggml_ops.grouped_mmq_gathered.default(
        input, row_index, packed_weight, expert_indices, expert_offsets, int(quant_type), int(out_features)
    )


def grouped_mmq_pair_gathered(
    input, row_index, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
) -> tuple[torch.Tensor, torch.Tensor]:
    """``grouped_mmq_pair(input.index_select(0, row_index), ...)`` without the sorted copy of the activations."""
    return torch.ops.torch_ggml_ops.grouped_mmq_pair_gathered.default(
        input, row_index, first_packed_weight, second_packed_weight, expert_indices, expert_offsets,
        int(quant_type), int(out_features),
    )


__all__ = ["grouped_mmq_gathered", "grouped_mmq_pair_gathered"]
