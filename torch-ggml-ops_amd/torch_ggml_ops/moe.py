"""The steps of a mixture-of-experts layer on either side of the grouped operators.

The reference's grouped operators start and end at expert-sorted rows and leave routing to the
caller (torch_ggml_ops/grouped_mmq.py:216).  This module holds the caller's side for this library:

* ``route``        sorts the (token, choice) slots by expert without a host synchronisation,
* ``moe_combine``  returns sorted rows to tokens, ``out[t] = sum_j w[t, j] * rows[slot_rows[t, j]]``,
                   in one deterministic pass (fp32 accumulation in choice order, one rounding),
* ``grouped_mmq_combine``  is the down projection followed by ``moe_combine`` as one differentiable step: its
                   backward folds the gather and the routing-weight scaling of the combine's gradient into the
                   packing of the down projection's cotangent, so the expert-sorted cotangent is never built,
* ``moe_layer``    chains gathered gate/up pair with fused SwiGLU -> down + combine.
"""

from __future__ import annotations

import torch

from . import _native, _validate
from .grouped_mmq import _forward as _grouped_forward
from .swiglu import grouped_mmq_swiglu

torch.library.define(
    "torch_ggml_ops::moe_combine", "(Tensor rows, Tensor slot_rows, Tensor slot_weights) -> Tensor"
)


def _fail(message: str) -> None:
    raise RuntimeError(message)


def _check_combine(rows: torch.Tensor, slot_rows: torch.Tensor, slot_weights: torch.Tensor) -> None:
    for tensor, name in ((rows, "rows"), (slot_rows, "slot_rows"), (slot_weights, "slot_weights")):
        if not tensor.is_cuda:
            _fail(f"{name} must be a CUDA/HIP tensor")
        if tensor.device != rows.device:
            _fail("all moe_combine tensors must be on the same device")
        if not tensor.is_contiguous():
            _fail(f"{name} must be contiguous; torch_ggml_ops will not insert a hidden copy")
    if rows.dtype != torch.bfloat16:
        _fail("rows must have dtype torch.bfloat16")
    if slot_rows.dtype != torch.int64:
        _fail("slot_rows must have dtype torch.int64")
    if slot_weights.dtype != torch.float32:
        _fail("slot_weights must have dtype torch.float32")
    if rows.dim() != 2 or rows.shape[0] <= 0:
        _fail("rows must have shape [rows, features] with at least one row")
    if slot_rows.dim() != 2 or slot_rows.shape != slot_weights.shape or slot_rows.numel() <= 0:
        _fail("slot_rows and slot_weights must both have shape [tokens, top_k]")
    if rows.shape[1] <= 0 or rows.shape[1] % 8 != 0:
        _fail(f"features must be a positive multiple of 8; got {rows.shape[1]}")
    if rows.data_ptr() % 16 != 0:
        _fail("rows data pointer must be 16-byte aligned")


def _combine_device(rows, slot_rows, slot_weights):
    _check_combine(rows, slot_rows, slot_weights)
    tokens, top_k = slot_rows.shape
    with _native.on_device(rows.device):
        output = rows.new_empty((tokens, rows.shape[1]))
        _native.check(
            _native.lib.tgo_moe_combine(
                rows.data_ptr(), slot_rows.data_ptr(), slot_weights.data_ptr(), output.data_ptr(),
                tokens, top_k, rows.shape[0], rows.shape[1], _native.stream_of(rows.device),
            )
        )
    return output


torch.library.impl("torch_ggml_ops::moe_combine", "CUDA")(_combine_device)


@torch.library.register_fake("torch_ggml_ops::moe_combine")
def _combine_fake(rows, slot_rows, slot_weights):
    return rows.new_empty((slot_rows.shape[0], rows.shape[1]))


def _setup_combine_context(ctx, inputs, output) -> None:
    rows, slot_rows, slot_weights = inputs
    ctx.num_rows = rows.shape[0]
    ctx.save_for_backward(rows if ctx.needs_input_grad[2] else None, slot_rows, slot_weights)


def _combine_backward(ctx, grad_output):
    rows, slot_rows, slot_weights = ctx.saved_tensors
    tokens, top_k = slot_rows.shape
    flat = slot_rows.reshape(-1)
    present = (flat >= 0) & (flat < ctx.num_rows)
    safe = flat.clamp(0, ctx.num_rows - 1)
    grad_per_slot = grad_output.repeat_interleave(top_k, dim=0)
    grad_rows = grad_weights = None
    if ctx.needs_input_grad[0]:
        scaled = (grad_per_slot.float() * (slot_weights.reshape(-1, 1) * present.unsqueeze(1))).to(grad_output.dtype)
        grad_rows = grad_output.new_zeros((ctx.num_rows, grad_output.shape[1]))
        # every row belongs to at most one slot, so this is a plain scatter, not a reduction
        grad_rows.index_add_(0, safe, scaled)
    if ctx.needs_input_grad[2]:
        products = (rows.index_select(0, safe).float() * grad_per_slot.float()).sum(dim=1)
        grad_weights = (products * present).reshape(tokens, top_k)
    return grad_rows, None, grad_weights


torch.library.register_autograd("torch_ggml_ops::moe_combine", _combine_backward, setup_context=_setup_combine_context)


def moe_combine(rows: torch.Tensor, slot_rows: torch.Tensor, slot_weights: torch.Tensor) -> torch.Tensor:
    """``out[t] = sum_j slot_weights[t, j] * rows[slot_rows[t, j]]``: bf16 rows, fp32 weights, bf16 result."""
    return torch.ops.torch_ggml_ops.moe_combine.default(rows, slot_rows, slot_weights)


torch.library.define(
    "torch_ggml_ops::grouped_mmq_grad_input_weighted",
    "(Tensor grad_tokens, Tensor row_token, Tensor row_weight, Tensor packed_weight, Tensor expert_indices, "
    "Tensor expert_offsets, int quant_type, int in_features) -> Tensor",
)
torch.library.define(
    "torch_ggml_ops::grouped_mmq_combine",
    "(Tensor input, Tensor packed_weight, Tensor expert_indices, Tensor expert_offsets, Tensor slot_rows, "
    "Tensor slot_weights, int quant_type, int out_features) -> (Tensor, Tensor)",
)


@torch.library.impl("torch_ggml_ops::grouped_mmq_grad_input_weighted", "CUDA")
def _grad_input_weighted_device(
    grad_tokens, row_token, row_weight, packed_weight, expert_indices, expert_offsets, quant_type, in_features
):
    shape = _validate.grouped(
        grad_tokens, packed_weight, expert_indices, expert_offsets, quant_type, in_features, backward=True
    )
    tokens, in_features, out_features, experts, groups, _bytes_per_expert = shape
    rows = _validate.row_index(row_token, grad_tokens)
    if row_weight.dtype != torch.float32 or row_weight.shape != row_token.shape or not row_weight.is_contiguous():
        _fail("row_weight must be a contiguous torch.float32 tensor with one entry per row")
    if row_weight.device != grad_tokens.device:
        _fail("all grouped MMQ backward tensors must be on the same device")
    with _native.on_device(grad_tokens.device):
        # (rows that no valid group covers stay unwritten, as for grouped_mmq_grad_input)
        grad_input = grad_tokens.new_empty((rows, in_features))
        workspace = grad_tokens.new_empty(
            (_native.lib.tgo_grad_workspace_bytes(rows, out_features, groups, 1),), dtype=torch.uint8
        )
        _native.check(
            _native.lib.tgo_grouped_mmq_grad_input_weighted(
                grad_tokens.data_ptr(), row_token.data_ptr(), row_weight.data_ptr(), tokens,
                packed_weight.data_ptr(), grad_input.data_ptr(), expert_indices.data_ptr(), expert_offsets.data_ptr(),
                workspace.data_ptr(), rows, out_features, in_features, experts, groups, int(quant_type),
                _native.stream_of(grad_tokens.device),
            )
        )
    return grad_input


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_grad_input_weighted")
def _grad_input_weighted_fake(
    grad_tokens, row_token, row_weight, packed_weight, expert_indices, expert_offsets, quant_type, in_features
):
    return grad_tokens.new_empty((row_token.shape[0], in_features))


@torch.library.impl("torch_ggml_ops::grouped_mmq_combine", "CUDA")
def _grouped_combine_device(
    input, packed_weight, expert_indices, expert_offsets, slot_rows, slot_weights, quant_type, out_features
):
    rows = _grouped_forward(input, packed_weight, None, expert_indices, expert_offsets, quant_type, out_features)[0]
    return _combine_device(rows, slot_rows, slot_weights), rows


@torch.library.register_fake("torch_ggml_ops::grouped_mmq_combine")
def _grouped_combine_fake(
    input, packed_weight, expert_indices, expert_offsets, slot_rows, slot_weights, quant_type, out_features
):
    return input.new_empty((slot_rows.shape[0], out_features)), input.new_empty((input.shape[0], out_features))


def _setup_grouped_combine_context(ctx, inputs, output) -> None:
    input, packed_weight, expert_indices, expert_offsets, slot_rows, slot_weights, quant_type, _out_features = inputs
    ctx.quant_type = quant_type
    ctx.num_rows, ctx.in_features = input.shape
    # (the second output, the expert-sorted rows, only serves the gradient of the routing weights: without this the
    # engine would hand the backward a zero tensor of its size)
    ctx.set_materialize_grads(False)
    ctx.save_for_backward(
        packed_weight, expert_indices, expert_offsets, slot_rows, slot_weights,
        output[1] if ctx.needs_input_grad[5] else None,
    )


def _grouped_combine_backward(ctx, grad_output, grad_rows):
    if grad_rows is not None:
        raise RuntimeError("grouped_mmq_combine: the expert-sorted rows are an auxiliary output without a gradient")
    packed_weight, expert_indices, expert_offsets, slot_rows, slot_weights, rows = ctx.saved_tensors
    if grad_output is None:
        return None, None, None, None, None, None, None, None
    tokens, top_k = slot_rows.shape
    flat = slot_rows.reshape(-1)
    present = (flat >= 0) & (flat < ctx.num_rows)
    safe = flat.clamp(0, ctx.num_rows - 1)
    grad_output = grad_output.contiguous()
    grad_input = grad_weights = None
    if ctx.needs_input_grad[0]:
        # the inverse of slot_rows: token and routing weight of every expert-sorted row (rows that no slot names
        # keep token -1, i.e. a zero cotangent); slots outside the rows are sent to a spare entry
        spare = ctx.num_rows
        target = torch.where(present, safe, torch.full_like(safe, spare))
        row_token = torch.full((ctx.num_rows + 1,), -1, dtype=torch.int64, device=flat.device)
        row_token[target] = torch.arange(tokens, device=flat.device).repeat_interleave(top_k)
        row_weight = torch.zeros((ctx.num_rows + 1,), dtype=torch.float32, device=flat.device)
        row_weight[target] = slot_weights.reshape(-1)
        grad_input = torch.ops.torch_ggml_ops.grouped_mmq_grad_input_weighted.default(
            grad_output, row_token[:spare].contiguous(), row_weight[:spare].contiguous(), packed_weight,
            expert_indices, expert_offsets, ctx.quant_type, ctx.in_features,
        )
    if ctx.needs_input_grad[5]:
        grad_per_slot = grad_output.repeat_interleave(top_k, dim=0)
        products = (rows.index_select(0, safe).float() * grad_per_slot.float()).sum(dim=1)
        grad_weights = (products * present).reshape(tokens, top_k)
    return grad_input, None, None, None, None, grad_weights, None, None


torch.library.register_autograd(
    "torch_ggml_ops::grouped_mmq_combine", _grouped_combine_backward, setup_context=_setup_grouped_combine_context
)


def grouped_mmq_combine(
    input: torch.Tensor,
    packed_weight: torch.Tensor,
    expert_indices: torch.Tensor,
    expert_offsets: torch.Tensor,
    slot_rows: torch.Tensor,
    slot_weights: torch.Tensor,
    quant_type: int,
    out_features: int,
) -> torch.Tensor:
    """``moe_combine(grouped_mmq(input, packed_weight, ...), slot_rows, slot_weights)`` as one differentiable step.

    Forward: the grouped projection of the expert-sorted ``input`` rows, then the routing-weighted return to
    tokens (bit-identical to the two separate calls).  Backward with respect to ``input``: the per-token gradient
    is gathered and scaled by the routing weight while the projection's cotangent is packed, so the
    expert-sorted gradient of the separate calls (``rows x out_features`` bf16 written, then read) never exists;
    the result equals theirs bit for bit.  Also differentiable with respect to ``slot_weights``.

    Every expert-sorted row may be named by at most one (token, choice) slot of ``slot_rows``, as ``route``
    guarantees: the backward inverts ``slot_rows`` into one (token, weight) per row, so a row named twice would keep
    one of its slots only, whereas the forward (and the separate ``moe_combine``) adds both.
    """
    output, _rows = torch.ops.torch_ggml_ops.grouped_mmq_combine.default(
        input, packed_weight, expert_indices, expert_offsets, slot_rows, slot_weights, int(quant_type), int(out_features)
    )
    return output


ROUTE_SMALL_LIMIT = 4096   # TGO_ROUTE_SMALL_LIMIT


torch.library.define(
    "torch_ggml_ops::route_small",
    "(Tensor slot_experts, int num_experts) -> (Tensor, Tensor, Tensor, Tensor)",
)


@torch.library.impl("torch_ggml_ops::route_small", "CUDA")
def _route_small_device(slot_experts, num_experts):
    """``route`` for a decode-sized batch as one kernel (``tgo_route_small``) instead of a sort and a dozen small
    tensor operations, which at that size cost more than the layer's own launches.  Same results."""
    slot_experts = slot_experts.to(torch.int64).contiguous()
    tokens, top_k = slot_experts.shape
    device = slot_experts.device
    row_index = torch.empty(tokens * top_k, dtype=torch.int64, device=device)
    slot_rows = torch.empty((tokens, top_k), dtype=torch.int64, device=device)
    expert_indices = torch.empty(num_experts, dtype=torch.int64, device=device)
    expert_offsets = torch.empty(num_experts, dtype=torch.int32, device=device)
    with _native.on_device(device):
        _native.check(
            _native.lib.tgo_route_small(
                slot_experts.data_ptr(), tokens, top_k, num_experts, row_index.data_ptr(), slot_rows.data_ptr(),
                expert_indices.data_ptr(), expert_offsets.data_ptr(), _native.stream_of(device),
            )
        )
    return row_index, slot_rows, expert_indices, expert_offsets


@torch.library.register_fake("torch_ggml_ops::route_small")
def _route_small_fake(slot_experts, num_experts):
    tokens, top_k = slot_experts.shape
    return (
        slot_experts.new_empty((tokens * top_k,), dtype=torch.int64),
        slot_experts.new_empty((tokens, top_k), dtype=torch.int64),
        slot_experts.new_empty((num_experts,), dtype=torch.int64),
        slot_experts.new_empty((num_experts,), dtype=torch.int32),
    )


def route(slot_experts: torch.Tensor, num_experts: int):
    """Sorts the ``[tokens, top_k]`` expert choices by expert (stable, no host synchronisation).

    Returns ``(row_index, slot_rows, expert_indices, expert_offsets)``: the token of each sorted row, the
    sorted row of each (token, choice) slot, and the group metadata of the grouped operators with one
    group per expert (experts without rows are empty groups, which the operators skip).
    """
    tokens, top_k = slot_experts.shape
    if slot_experts.is_cuda and 0 < tokens * top_k <= ROUTE_SMALL_LIMIT and 0 < num_experts <= ROUTE_SMALL_LIMIT:
        return torch.ops.torch_ggml_ops.route_small.default(slot_experts, int(num_experts))
    flat = slot_experts.reshape(-1)
    order = torch.argsort(flat, stable=True)
    row_index = torch.div(order, top_k, rounding_mode="floor")
    slot_rows = torch.empty_like(order)
    slot_rows[order] = torch.arange(order.numel(), device=order.device)
    counts = torch.zeros(num_experts, dtype=torch.int64, device=flat.device)
    counts.scatter_add_(0, flat, torch.ones_like(flat))
    expert_offsets = counts.cumsum(0).to(torch.int32)
    expert_indices = torch.arange(num_experts, dtype=torch.int64, device=flat.device)
    return row_index, slot_rows.reshape(tokens, top_k), expert_indices, expert_offsets


def moe_layer(
    hidden: torch.Tensor,
    slot_experts: torch.Tensor,
    slot_weights: torch.Tensor,
    gate_weight: torch.Tensor,
    up_weight: torch.Tensor,
    down_weight: torch.Tensor,
    gate_up_type: int,
    down_type: int,
    intermediate_features: int,
) -> torch.Tensor:
    """SwiGLU mixture-of-experts layer over packed expert weights.

    ``hidden`` bf16 ``[tokens, features]``; ``slot_experts`` int64 and ``slot_weights`` fp32
    ``[tokens, top_k]``; ``gate_weight``/``up_weight`` packed ``[experts, intermediate, ...]`` and
    ``down_weight`` packed ``[experts, features, ...]``.  Differentiable with respect to ``hidden`` and
    ``slot_weights``.
    """
    experts = gate_weight.shape[0]
    row_index, slot_rows, expert_indices, expert_offsets = route(slot_experts, experts)
    activated = grouped_mmq_swiglu(
        hidden, gate_weight, up_weight, expert_indices, expert_offsets, gate_up_type, intermediate_features, row_index
    )
    return grouped_mmq_combine(
        activated, down_weight, expert_indices, expert_offsets, slot_rows, slot_weights, down_type, hidden.shape[1]
    )


__all__ = ["grouped_mmq_combine", "moe_combine", "moe_layer", "route"]
