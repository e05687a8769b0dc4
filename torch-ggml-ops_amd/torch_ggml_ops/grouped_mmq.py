"""Grouped (mixture-of-experts) packed-GGUF matmul over expert-sorted rows.

Same operator surface as the reference (torch_ggml_ops/grouped_mmq.py:1-250 and the
schemas at csrc/mmq_hip.cu:1202-1214).  Group ``g`` covers rows
``[expert_offsets[g-1], expert_offsets[g])`` and uses the weights of expert
``expert_indices[g]``; rows outside every valid group are left uninitialised.
"""

from __future__ import annotations

import torch

from . import _native, _validate

torch.library.define(
    "torch_ggml_ops::grouped_mmq_grad_input",
    "(Tensor grad_output, Tensor packed_weight, Tensor expert_indices, Tensor expert_offsets, "
    "int quant_type, int in_features) -> Tensor",
)
torch.library.define(
    "torch_ggml_ops::grouped_mmq_pair_grad_input",
    "(Tensor first_grad_output, Tensor second_grad_output, Tensor first_packed_weight, "
    "Tensor second_packed_weight, Tensor expert_indices, Tensor expert_offsets, int quant_type, "
    "int in_features) -> Tensor",
)
torch.library.define(
    "torch_ggml_ops::grouped_mmq",
    "(Tensor input, Tensor packed_weight, Tensor expert_indices, Tensor expert_offsets, "
    "int quant_type, int out_features) -> Tensor",
)
torch.library.define(
    "torch_ggml_ops::grouped_mmq_pair",
    "(Tensor input, Tensor first_packed_weight, Tensor second_packed_weight, Tensor expert_indices, "
    "Tensor expert_offsets, int quant_type, int out_features) -> (Tensor, Tensor)",
)


def _stream(tensor: torch.Tensor) -> int:
    return _native.stream_of(tensor.device)


def _forward(
    input, first_weight, second_weight, expert_indices, expert_offsets, quant_type, out_features, row_index=None,
    swiglu=False,
):
    """Grouped forward; with ``row_index`` operator row ``r`` is ``input[row_index[r]]`` (gathered while quantizing).
    With ``swiglu`` (pair only) the second result is ``silu(first) * second`` from the kernel's epilogue."""
    shape = _validate.grouped(input, first_weight, expert_indices, expert_offsets, quant_type, out_features, backward=False)
    rows, in_features, out_features, experts, groups, bytes_per_expert = shape
    input_rows = rows
    if row_index is not None:
        rows = _validate.row_index(row_index, input)
    if second_weight is not None and not _validate.same_weight_geometry(first_weight, second_weight):
        second = _validate.grouped(
            input, second_weight, expert_indices, expert_offsets, quant_type, out_features, backward=False
        )
        if second[3] != experts or second[5] != bytes_per_expert:
            raise RuntimeError("paired grouped MMQ weights must have identical physical geometry")
    with _native.on_device(input.device):
        first_output = input.new_empty((rows, out_features))
        second_output = input.new_empty((rows, out_features)) if second_weight is not None else None
        workspace_bytes = (
            _native.lib.tgo_q8_workspace_bytes(rows, in_features) + _native.lib.tgo_task_workspace_bytes(rows, groups)
        )
        workspace = input.new_empty((workspace_bytes,), dtype=torch.uint8)
        gather = () if row_index is None else (row_index.data_ptr(), input_rows)
        entry = _native.lib.tgo_grouped_mmq_forward if row_index is None else _native.lib.tgo_grouped_mmq_forward_gathered
        if swiglu:
            gather = (row_index.data_ptr() if row_index is not None else None, input_rows)
            entry = _native.lib.tgo_grouped_mmq_swiglu
        _native.check(
            entry(
                input.data_ptr(),
                *gather,
                first_weight.data_ptr(),
                second_weight.data_ptr() if second_weight is not None else None,
                first_output.data_ptr(),
                second_output.data_ptr() if second_output is not None else None,
                expert_indices.data_ptr(),
                expert_offsets.data_ptr(),
                workspace.data_ptr(),
                rows, in_features, out_features, experts, groups, int(quant_type), _stream(input),
            )
        )
    return first_output, second_output


def _grad_input(
    first_grad, second_grad, first_weight, second_weight, expert_indices, expert_offsets, quant_type, in_features,
    zero_fill=False,
):
    """Grouped grad-input; ``zero_fill`` clears the rows that no valid group covers (they stay unwritten otherwise)."""
    shape = _validate.grouped(first_grad, first_weight, expert_indices, expert_offsets, quant_type, in_features, backward=True)
    rows, in_features, out_features, experts, groups, bytes_per_expert = shape
    if second_weight is not None:
        second = _validate.grouped(
            second_grad, second_weight, expert_indices, expert_offsets, quant_type, in_features, backward=True
        )
        if (second[0], second[2], second[3], second[4], second[5]) != (rows, out_features, experts, groups, bytes_per_expert):
            raise RuntimeError("paired grouped MMQ backward tensors must have identical physical geometry")
    with _native.on_device(first_grad.device):
        grad_input = (first_grad.new_zeros if zero_fill else first_grad.new_empty)((rows, in_features))
        sources = 2 if second_weight is not None else 1
        workspace = first_grad.new_empty(
            (_native.lib.tgo_grad_workspace_bytes(rows, out_features, groups, sources),), dtype=torch.uint8
        )
        _native.check(
            _native.lib.tgo_grouped_mmq_grad_input(
                first_grad.data_ptr(),
                second_grad.data_ptr() if second_grad is not None else None,
                first_weight.data_ptr(),
                second_weight.data_ptr() if second_weight is not None else None,
                grad_input.data_ptr(),
                expert_indices.data_ptr(),
                expert_offsets.data_ptr(),
                workspace.data_ptr(),
                rows, out_features, in_features, experts, groups, int(quant_type), _stream(first_grad),
            )
        )
    return grad_input


@torch.library.impl("torch_ggml_ops::grouped_mmq", "CUDA")
def _grouped_mmq_device(input, packed_weight, expert_indices, expert_offsets, quant_type, out_features):
    return _forward(input, packed_weight, None, expert_indices, expert_offsets, quant_type, out_features)[0]


@torch.library.impl("torch_ggml_ops::grouped_mmq_pair", "CUDA")
def _grouped_mmq_pair_device(
    input, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
):
    return _forward(
        input, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
    )


@torch.library.impl("torch_ggml_ops::grouped_mmq_grad_input", "CUDA")
def _grouped_mmq_grad_input_device(grad_output, packed_weight, expert_indices, expert_offsets, quant_type, in_features):
    return _grad_input(grad_output, None, packed_weight, None, expert_indices, expert_offsets, quant_type, in_features)


@torch.library.impl("torch_ggml_ops::grouped_mmq_pair_grad_input", "CUDA")
def _grouped_mmq_pair_grad_input_device(
    first_grad_output, second_grad_output, first_packed_weight, second_packed_weight,
    expert_indices, expert_offsets, quant_type, in_features,
):
    return _grad_input(
        first_grad_output, second_grad_output, first_packed_weight, second_packed_weight,
        expert_indices, expert_offsets, quant_type, in_features,
    )


@torch.library.register_fake("torch_ggml_ops::grouped_mmq")
def _grouped_mmq_fake(input, packed_weight, expert_indices, expert_offsets, quant_type, out_features):
    return input.new_empty((input.shape[0], out_features))


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_grad_input")
def _grouped_mmq_grad_input_fake(grad_output, packed_weight, expert_indices, expert_offsets, quant_type, in_features):
    return grad_output.new_empty((grad_output.shape[0], in_features))


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_pair_grad_input")
def _grouped_mmq_pair_grad_input_fake(
    first_grad_output, second_grad_output, first_packed_weight, second_packed_weight,
    expert_indices, expert_offsets, quant_type, in_features,
):
    return first_grad_output.new_empty((first_grad_output.shape[0], in_features))


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_pair")
def _grouped_mmq_pair_fake(
    input, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
):
    shape = (input.shape[0], out_features)
    return input.new_empty(shape), input.new_empty(shape)


def _single_grad_input(grad_output, packed_weight, expert_indices, expert_offsets, quant_type, in_features):
    return torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(
        grad_output.contiguous(), packed_weight, expert_indices, expert_offsets, quant_type, in_features
    )


def _setup_grouped_context(ctx, inputs, output) -> None:
    input, packed_weight, expert_indices, expert_offsets, quant_type, _out_features = inputs
    ctx.quant_type = quant_type
    ctx.in_features = input.shape[1]
    if ctx.needs_input_grad[0]:
        ctx.save_for_backward(packed_weight, expert_indices, expert_offsets)


def _grouped_backward(ctx, grad_output: torch.Tensor):
    grad_input = None
    if ctx.needs_input_grad[0]:
        packed_weight, expert_indices, expert_offsets = ctx.saved_tensors
        grad_input = _single_grad_input(
            grad_output, packed_weight, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
        )
    return grad_input, None, None, None, None, None


torch.library.register_autograd("torch_ggml_ops::grouped_mmq", _grouped_backward, setup_context=_setup_grouped_context)


def _no_double_backward(name: str):
    def backward(ctx, grad_grad_input: torch.Tensor):
        raise RuntimeError(f"torch_ggml_ops::{name} does not support higher-order gradients")

    return backward


torch.library.register_autograd(
    "torch_ggml_ops::grouped_mmq_grad_input", _no_double_backward("grouped_mmq_grad_input")
)
torch.library.register_autograd(
    "torch_ggml_ops::grouped_mmq_pair_grad_input", _no_double_backward("grouped_mmq_pair_grad_input")
)


def _setup_pair_context(ctx, inputs, output) -> None:
    input, first_weight, second_weight, expert_indices, expert_offsets, quant_type, _out_features = inputs
    ctx.quant_type = quant_type
    ctx.in_features = input.shape[1]
    if ctx.needs_input_grad[0]:
        ctx.save_for_backward(first_weight, second_weight, expert_indices, expert_offsets)


def _pair_backward(ctx, first_grad_output, second_grad_output):
    grad_input = None
    if ctx.needs_input_grad[0]:
        first_weight, second_weight, expert_indices, expert_offsets = ctx.saved_tensors
        if first_grad_output is not None and second_grad_output is not None:
            grad_input = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
                first_grad_output.contiguous(), second_grad_output.contiguous(), first_weight, second_weight,
                expert_indices, expert_offsets, ctx.quant_type, ctx.in_features,
            )
        elif first_grad_output is not None:
            grad_input = _single_grad_input(
                first_grad_output, first_weight, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
            )
        elif second_grad_output is not None:
            grad_input = _single_grad_input(
                second_grad_output, second_weight, expert_indices, expert_offsets, ctx.quant_type, ctx.in_features
            )
    return grad_input, None, None, None, None, None, None


torch.library.register_autograd("torch_ggml_ops::grouped_mmq_pair", _pair_backward, setup_context=_setup_pair_context)


def grouped_mmq(input, packed_weight, expert_indices, expert_offsets, quant_type, out_features) -> torch.Tensor:
    """Grouped packed GGUF matmul over expert-sorted bf16 rows."""
    return torch.ops.torch_ggml_ops.grouped_mmq.default(
        input, packed_weight, expert_indices, expert_offsets, int(quant_type), int(out_features)
    )


def grouped_mmq_pair(
    input, first_packed_weight, second_packed_weight, expert_indices, expert_offsets, quant_type, out_features
) -> tuple[torch.Tensor, torch.Tensor]:
    """Two grouped projections (gate and up) that share one q8_1 activation workspace."""
    return torch.ops.torch_ggml_ops.grouped_mmq_pair.default(
        input, first_packed_weight, second_packed_weight, expert_indices, expert_offsets,
        int(quant_type), int(out_features),
    )


__all__ = ["grouped_mmq", "grouped_mmq_pair"]
