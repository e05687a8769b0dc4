"""Dense packed-GGUF matmul: ``mmq`` and its grad-input operator.

Same operator surface as the reference (torch_ggml_ops/mmq.py:1-83 and the schemas at
csrc/mmq_hip.cu:1197-1201): bf16 activations, raw GGUF blocks as uint8, gradient with
respect to the input only.  The device implementations call the gfx950 library through
its C ABI on the caller's current stream.
"""

from __future__ import annotations

import torch

from . import _native, _validate

torch.library.define(
    "torch_ggml_ops::mmq",
    "(Tensor input, Tensor packed_weight, int quant_type, int out_features) -> Tensor",
)
torch.library.define(
    "torch_ggml_ops::mmq_grad_input",
    "(Tensor grad_output, Tensor packed_weight, int quant_type, int in_features) -> Tensor",
)


def _stream(tensor: torch.Tensor) -> int:
    return _native.stream_of(tensor.device)


@torch.library.impl("torch_ggml_ops::mmq", "CUDA")
def _mmq_device(input: torch.Tensor, packed_weight: torch.Tensor, quant_type: int, out_features: int) -> torch.Tensor:
    rows, in_features, out_features = _validate.dense(input, packed_weight, quant_type, out_features, backward=False)
    with _native.on_device(input.device):
        output = input.new_empty((*input.shape[:-1], out_features))
        workspace = input.new_empty(
            (_native.lib.tgo_q8_workspace_bytes(rows, in_features),), dtype=torch.uint8
        )
        _native.check(
            _native.lib.tgo_mmq_forward(
                input.data_ptr(), packed_weight.data_ptr(), output.data_ptr(), workspace.data_ptr(),
                rows, in_features, out_features, int(quant_type), _stream(input),
            )
        )
    return output


@torch.library.impl("torch_ggml_ops::mmq_grad_input", "CUDA")
def _mmq_grad_input_device(
    grad_output: torch.Tensor, packed_weight: torch.Tensor, quant_type: int, in_features: int
) -> torch.Tensor:
    rows, in_features, out_features = _validate.dense(grad_output, packed_weight, quant_type, in_features, backward=True)
    with _native.on_device(grad_output.device):
        grad_input = grad_output.new_empty((*grad_output.shape[:-1], in_features))
        workspace = grad_output.new_empty(
            (_native.lib.tgo_dense_grad_workspace_bytes(rows, out_features, in_features, quant_type),), dtype=torch.uint8
        )
        _native.check(
            _native.lib.tgo_mmq_grad_input(
                grad_output.data_ptr(), packed_weight.data_ptr(), grad_input.data_ptr(), workspace.data_ptr(),
                rows, out_features, in_features, int(quant_type), _stream(grad_output),
            )
        )
    return grad_input


@torch.library.register_fake("torch_ggml_ops::mmq")
def _mmq_fake(input, packed_weight, quant_type, out_features):
    return input.new_empty((*input.shape[:-1], out_features))


@torch.library.register_fake("torch_ggml_ops::mmq_grad_input")
def _mmq_grad_input_fake(grad_output, packed_weight, quant_type, in_features):
    return grad_output.new_empty((*grad_output.shape[:-1], in_features))


def _setup_mmq_context(ctx, inputs, output) -> None:
    input, packed_weight, quant_type, _out_features = inputs
    ctx.quant_type = quant_type
    ctx.in_features = input.shape[-1]
    if ctx.needs_input_grad[0]:
        ctx.save_for_backward(packed_weight)


def _mmq_backward(ctx, grad_output: torch.Tensor):
    grad_input = None
    if ctx.needs_input_grad[0]:
        (packed_weight,) = ctx.saved_tensors
        # autograd may hand over a non-contiguous cotangent; the operator itself never copies
        grad_input = torch.ops.torch_ggml_ops.mmq_grad_input.default(
            grad_output.contiguous(), packed_weight, ctx.quant_type, ctx.in_features
        )
    return grad_input, None, None, None


torch.library.register_autograd("torch_ggml_ops::mmq", _mmq_backward, setup_context=_setup_mmq_context)


def _mmq_grad_input_backward(ctx, grad_grad_input: torch.Tensor):
    raise RuntimeError("torch_ggml_ops::mmq_grad_input does not support higher-order gradients")


torch.library.register_autograd("torch_ggml_ops::mmq_grad_input", _mmq_grad_input_backward)


def mmq(input: torch.Tensor, packed_weight: torch.Tensor, quant_type: int, out_features: int) -> torch.Tensor:
    """``input @ W.T`` for a packed GGUF weight ``[out_features, row_bytes]``; bf16 in, bf16 out."""
    return torch.ops.torch_ggml_ops.mmq.default(input, packed_weight, int(quant_type), int(out_features))


__all__ = ["mmq"]
