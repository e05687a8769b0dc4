"""Several dense projections of one input: quantize the activations once, multiply many times.

``mmq`` quantizes its input to q8_1 blocks on every call.  When the same activations feed
several packed weights (q/k/v, a shared expert's gate/up), that work and its HBM traffic can be
paid once: ``quantize_q8_1`` returns the library's q8_1 workspace as an opaque uint8 tensor and
``mmq_prepared`` runs only the matmul half on it.  A workspace that is quantized before its format is
known holds int8 operands (exact fp16 ones when ``set_forward_operand("half")`` forces them), so the
results are bit-identical to ``mmq`` wherever ``mmq`` multiplies the same kind: formats other than IQ2_S
in calls below the size at which ``mmq`` switches to its scaled operands (``forward_operand_for``).
Otherwise they are the same q8_1 algebra with another summation order or operand rounding (IQ2_S: exact
fp16 in ``mmq``, int8 here, whose kernel is about a third slower for that format; large calls: scaled
operands in ``mmq``, up to 8e-4 of the largest output apart).  A caller that knows what the workspace
will be multiplied with names the kind itself (``operand=`` of both functions, the same value in both);
``mmq_multi`` does, from the formats and the summed width of its projections, so q/k/v of a long
sequence run on the scaled kernels like one large ``mmq``.

The reference has no such operator; it lists this reuse as its next optimisation
(docs/mmq_fwd_optimization.md:299-307).  ``mmq_multi`` is the convenience wrapper with autograd
(gradient with respect to the input only, as for ``mmq``: the sum of the projections'
``mmq_grad_input``).
"""

from __future__ import annotations

from typing import Sequence

import torch

from . import _native, _validate

torch.library.define("torch_ggml_ops::quantize_q8_1", '(Tensor input, str operand="") -> Tensor')
torch.library.define(
    "torch_ggml_ops::mmq_prepared",
    "(Tensor workspace, Tensor packed_weight, int rows, int in_features, int quant_type, int out_features, "
    'str operand="") -> Tensor',
)


def _stream(tensor: torch.Tensor) -> int:
    return _native.stream_of(tensor.device)


def _workspace_kind(operand: str) -> int:
    """Operand kind of a workspace: the named one, or what the process-wide setting gives an unknown format."""
    if operand == "":
        return _native.lib.tgo_forward_operand_for(0, 0, 0, 1)
    if operand not in ("int8", "half", "scaled"):
        raise ValueError(f'operand must be "int8", "half", "scaled" or "" (by the setting); got {operand!r}')
    return _native.OPERANDS[operand]


def _activation_shape(input: torch.Tensor) -> tuple[int, int]:
    _validate.activation(input, "input")
    in_features = int(input.shape[-1])
    return input.numel() // in_features, in_features


@torch.library.impl("torch_ggml_ops::quantize_q8_1", "CUDA")
def _quantize_device(input: torch.Tensor, operand: str = "") -> torch.Tensor:
    rows, in_features = _activation_shape(input)
    kind = _workspace_kind(operand)
    with _native.on_device(input.device):
        workspace = input.new_empty((_native.lib.tgo_q8_workspace_bytes(rows, in_features),), dtype=torch.uint8)
        _native.check(
            _native.lib.tgo_quantize_q8_1_as(
                input.data_ptr(), workspace.data_ptr(), rows, in_features, kind, _stream(input)
            )
        )
    return workspace


@torch.library.register_fake("torch_ggml_ops::quantize_q8_1")
def _quantize_fake(input, operand=""):
    # (tgo_q8_workspace_bytes: two bytes per value, two fp32 per 32 values, 20 bytes per 256 values, 4 per row, 1 KiB)
    in_features = input.shape[-1]
    rows = input.numel() // in_features
    padded = (rows + 31) // 32 * 32
    size = 2 * padded * in_features + 8 * padded * (in_features // 32) + 20 * padded * (in_features // 256) + 4 * padded + 1024
    return input.new_empty((size,), dtype=torch.uint8)


@torch.library.impl("torch_ggml_ops::mmq_prepared", "CUDA")
def _mmq_prepared_device(
    workspace: torch.Tensor, packed_weight: torch.Tensor, rows: int, in_features: int, quant_type: int,
    out_features: int, operand: str = "",
) -> torch.Tensor:
    _validate.prepared(workspace, packed_weight, rows, in_features, quant_type, out_features)
    kind = _workspace_kind(operand)
    expected = _native.lib.tgo_q8_workspace_bytes(rows, in_features)
    if workspace.numel() != expected:
        raise RuntimeError(
            f"workspace holds {workspace.numel()} bytes; quantize_q8_1 of [{rows}, {in_features}] writes {expected}"
        )
    with _native.on_device(workspace.device):
        output = workspace.new_empty((rows, out_features), dtype=torch.bfloat16)
        _native.check(
            _native.lib.tgo_mmq_forward_prepared_as(
                workspace.data_ptr(), packed_weight.data_ptr(), output.data_ptr(),
                rows, in_features, out_features, int(quant_type), kind, _stream(workspace),
            )
        )
    return output


@torch.library.register_fake("torch_ggml_ops::mmq_prepared")
def _mmq_prepared_fake(workspace, packed_weight, rows, in_features, quant_type, out_features, operand=""):
    return workspace.new_empty((rows, out_features), dtype=torch.bfloat16)


class _MultiProjection(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, quant_types, out_features, *packed_weights):
        rows, in_features = _activation_shape(input)
        operand = multi_operand(quant_types, rows, out_features)
        workspace = torch.ops.torch_ggml_ops.quantize_q8_1.default(input, operand)
        outputs = tuple(
            torch.ops.torch_ggml_ops.mmq_prepared.default(
                workspace, weight, rows, in_features, int(quant_type), int(features), operand
            ).view(*input.shape[:-1], int(features))
            for weight, quant_type, features in zip(packed_weights, quant_types, out_features)
        )
        ctx.quant_types = tuple(int(q) for q in quant_types)
        ctx.in_features = in_features
        ctx.save_for_backward(*packed_weights)
        return outputs

    @staticmethod
    def backward(ctx, *grad_outputs):
        grad_input = None
        if ctx.needs_input_grad[0]:
            for grad, weight, quant_type in zip(grad_outputs, ctx.saved_tensors, ctx.quant_types):
                if grad is None:
                    continue
                term = torch.ops.torch_ggml_ops.mmq_grad_input.default(
                    grad.contiguous(), weight, quant_type, ctx.in_features
                )
                grad_input = term if grad_input is None else grad_input + term
        return (grad_input, None, None) + (None,) * len(ctx.saved_tensors)


def multi_operand(quant_types: Sequence[int], rows: int, out_features: Sequence[int]) -> str:
    """The operand kind for one workspace that feeds all these projections of ``rows`` activations.

    What ``mmq`` would take for one weight as wide as all of them together; int8, which every format's kernels
    read, when the formats disagree.
    """
    total = sum(int(features) for features in out_features)
    kinds = {_native.forward_operand_for(int(quant_type), int(rows), total) for quant_type in quant_types}
    return kinds.pop() if len(kinds) == 1 else "int8"


def quantize_q8_1(input: torch.Tensor, operand: str = "") -> torch.Tensor:
    """q8_1 workspace of ``input`` (bf16, last dimension a multiple of 256) for ``mmq_prepared``.

    ``operand``: "int8", "half" or "scaled" operands, or "" for what the process-wide setting gives a
    workspace of unknown use (int8 unless "half" is forced).
    """
    return torch.ops.torch_ggml_ops.quantize_q8_1.default(input, operand)


def mmq_prepared(
    workspace: torch.Tensor, packed_weight: torch.Tensor, rows: int, in_features: int, quant_type: int,
    out_features: int, operand: str = "",
) -> torch.Tensor:
    """``[rows, out_features]`` product of the activations behind ``workspace`` with one packed weight.

    ``operand`` must be what ``quantize_q8_1`` was given for this workspace; the output is NaN when it is not.
    """
    return torch.ops.torch_ggml_ops.mmq_prepared.default(
        workspace, packed_weight, int(rows), int(in_features), int(quant_type), int(out_features), operand
    )


def mmq_multi(
    input: torch.Tensor,
    packed_weights: Sequence[torch.Tensor],
    quant_types: Sequence[int],
    out_features: Sequence[int],
) -> tuple[torch.Tensor, ...]:
    """``tuple(mmq(input, w, q, n) for ...)`` with the activations quantized once."""
    if not (len(packed_weights) == len(quant_types) == len(out_features)) or not packed_weights:
        raise ValueError("packed_weights, quant_types and out_features must be non-empty and of equal length")
    return _MultiProjection.apply(input, tuple(quant_types), tuple(out_features), *packed_weights)


__all__ = ["mmq_multi", "mmq_prepared", "multi_operand", "quantize_q8_1"]
