"""Argument checks of the six operators.

Mirrors the reference's host-side validation (csrc/mmq_hip.cu:325-519, :587-631,
:680-739): fail fast with the same messages and never insert a hidden copy.
"""

from __future__ import annotations

import torch

from . import _native

QK_K = 256
_INT_MAX = 2**31 - 1


def _fail(message: str) -> None:
    raise RuntimeError(message)


def packed_block_bytes(quant_type: int) -> int:
    size = _native.lib.tgo_block_bytes(int(quant_type))
    if size == 0:
        _fail(f"unsupported quant_type: {quant_type}")
    return size


# The device checks can be switched off so that the remaining rules are testable on a host without a GPU.
REQUIRE_DEVICE = True


def _check_tensor(tensor: torch.Tensor, name: str, dtype: torch.dtype, dtype_name: str) -> None:
    if REQUIRE_DEVICE and not tensor.is_cuda:
        _fail(f"{name} must be a CUDA/HIP tensor")
    if tensor.dtype != dtype:
        _fail(f"{name} must have dtype {dtype_name}")


def _check_layout(tensor: torch.Tensor, name: str) -> None:
    if not tensor.is_contiguous():
        _fail(f"{name} must be contiguous; torch_ggml_ops will not insert a hidden copy")
    if tensor.storage_offset() != 0:
        _fail(f"{name} must have zero storage offset")


def _check_aligned(tensor: torch.Tensor, name: str) -> None:
    if tensor.data_ptr() % 16 != 0:
        _fail(f"{name} data pointer must be 16-byte aligned")


def dense(activation: torch.Tensor, packed_weight: torch.Tensor, quant_type: int, other_features: int, *, backward: bool):
    """Checks for mmq (activation = input, other = out_features) and mmq_grad_input
    (activation = grad_output, other = in_features).  Returns (rows, in_features, out_features)."""
    name = "grad_output" if backward else "input"
    _check_tensor(activation, name, torch.bfloat16, "torch.bfloat16")
    _check_tensor(packed_weight, "packed_weight", torch.uint8, "torch.uint8")
    if activation.device != packed_weight.device:
        _fail(f"{name} and packed_weight must be on the same device")
    if not activation.is_contiguous():
        _fail(f"{name} must be contiguous; torch_ggml_ops will not insert a hidden copy")
    if not packed_weight.is_contiguous():
        _fail("packed_weight must be contiguous; torch_ggml_ops will not insert a hidden copy")
    if activation.dim() < 1:
        _fail(f"{name} must have at least one dimension")
    if activation.storage_offset() != 0:
        _fail(f"{name} must have zero storage offset")
    if packed_weight.storage_offset() != 0:
        _fail("packed_weight must have zero storage offset")

    last = activation.shape[-1]
    if backward:
        in_features, out_features = int(other_features), int(last)
        if in_features <= 0 or in_features % QK_K != 0:
            _fail(f"in_features must be a positive multiple of 256; got {in_features}")
        if out_features <= 0:
            _fail("grad_output final dimension must be positive")
        rows = activation.numel() // out_features
        if rows <= 0:
            _fail("zero-row grad_output tensors are not supported")
        if rows > _INT_MAX:
            _fail("flattened grad_output row count exceeds the kernel limit")
    else:
        in_features, out_features = int(last), int(other_features)
        if in_features <= 0 or in_features % QK_K != 0:
            _fail(f"input width must be a positive multiple of 256; got {in_features}")
        if out_features <= 0:
            _fail(f"out_features must be positive; got {out_features}")
        rows = activation.numel() // in_features
        if rows <= 0:
            _fail("zero-row inputs are not supported")
        if rows > _INT_MAX:
            _fail("flattened input row count exceeds the kernel limit")
    if in_features > _INT_MAX:
        _fail("in_features exceeds the kernel limit")
    if out_features > _INT_MAX:
        _fail("out_features exceeds the kernel limit")

    expected = out_features * (in_features // QK_K) * packed_block_bytes(quant_type)
    if packed_weight.numel() != expected:
        _fail(
            f"packed_weight has {packed_weight.numel()} bytes, expected {expected} for "
            f"[{out_features}, {in_features}] quant_type={quant_type}"
        )
    _check_aligned(activation, name)
    _check_aligned(packed_weight, "packed_weight")
    return rows, in_features, out_features


def grouped(
    activation: torch.Tensor,
    packed_weight: torch.Tensor,
    expert_indices: torch.Tensor,
    expert_offsets: torch.Tensor,
    quant_type: int,
    other_features: int,
    *,
    backward: bool,
):
    """Checks for the grouped operators.  Returns (rows, in_features, out_features, experts, groups, bytes_per_expert)."""
    name = "grad_output" if backward else "input"
    _check_tensor(activation, name, torch.bfloat16, "torch.bfloat16")
    _check_tensor(packed_weight, "packed_weight", torch.uint8, "torch.uint8")
    if REQUIRE_DEVICE and not expert_indices.is_cuda:
        _fail("expert_indices must be a CUDA/HIP tensor")
    if REQUIRE_DEVICE and not expert_offsets.is_cuda:
        _fail("expert_offsets must be a CUDA/HIP tensor")
    device = activation.device
    if packed_weight.device != device or expert_indices.device != device or expert_offsets.device != device:
        _fail("all grouped MMQ backward tensors must be on the same device" if backward
              else "all grouped MMQ tensors must be on the same device")
    if expert_indices.dtype != torch.int64:
        _fail("expert_indices must have dtype torch.int64")
    if expert_offsets.dtype != torch.int32:
        _fail("expert_offsets must have dtype torch.int32")
    for tensor, label in (
        (activation, name),
        (packed_weight, "packed_weight"),
        (expert_indices, "expert_indices"),
        (expert_offsets, "expert_offsets"),
    ):
        if not tensor.is_contiguous():
            _fail(f"{label} must be contiguous; torch_ggml_ops will not insert a hidden copy")
    for tensor, label in (
        (activation, name),
        (packed_weight, "packed_weight"),
        (expert_indices, "expert_indices"),
        (expert_offsets, "expert_offsets"),
    ):
        if tensor.storage_offset() != 0:
            _fail(f"{label} must have zero storage offset")
    if activation.dim() != 2:
        _fail("grouped MMQ grad_output must have shape [rows, out_features]" if backward
              else "grouped MMQ input must have shape [rows, in_features]")
    if packed_weight.dim() != 3:
        _fail("grouped packed_weight must have physical shape [experts, out_features, row_bytes]")
    if expert_indices.dim() != 1:
        _fail("expert_indices must be one-dimensional")
    if expert_offsets.dim() != 1:
        _fail("expert_offsets must be one-dimensional")
    if expert_indices.numel() != expert_offsets.numel():
        _fail("expert_indices and expert_offsets must have equal lengths")
    if expert_indices.numel() <= 0:
        _fail("grouped MMQ backward requires at least one active expert" if backward
              else "grouped MMQ requires at least one active expert")

    rows = activation.shape[0]
    experts = packed_weight.shape[0]
    groups = expert_indices.numel()
    if backward:
        in_features, out_features = int(other_features), int(activation.shape[1])
        if rows <= 0:
            _fail("zero-row grad_output tensors are not supported")
        if out_features <= 0:
            _fail("grad_output final dimension must be positive")
        if in_features <= 0 or in_features % QK_K != 0:
            _fail(f"in_features must be a positive multiple of 256; got {in_features}")
    else:
        in_features, out_features = int(activation.shape[1]), int(other_features)
        if rows <= 0:
            _fail("zero-row inputs are not supported")
        if in_features <= 0 or in_features % QK_K != 0:
            _fail(f"input width must be a positive multiple of 256; got {in_features}")
        if out_features <= 0:
            _fail(f"out_features must be positive; got {out_features}")
    if experts <= 0:
        _fail("packed_weight must contain at least one expert")
    if groups > experts:
        _fail("active expert count exceeds packed expert count")
    if rows > _INT_MAX:
        _fail(f"{name} row count exceeds the kernel limit")
    if in_features > _INT_MAX:
        _fail("in_features exceeds the kernel limit")
    if out_features > _INT_MAX:
        _fail("out_features exceeds the kernel limit")
    if experts > _INT_MAX:
        _fail("expert count exceeds the kernel limit")

    row_bytes = (in_features // QK_K) * packed_block_bytes(quant_type)
    if packed_weight.shape[1] != out_features:
        _fail("packed_weight physical output dimension does not match grad_output" if backward
              else "packed_weight physical output dimension does not match out_features")
    if packed_weight.shape[2] != row_bytes:
        _fail(
            f"packed_weight has {packed_weight.shape[2]} bytes per row, expected {row_bytes} for "
            f"in_features={in_features} quant_type={quant_type}"
        )
    bytes_per_expert = out_features * row_bytes
    if packed_weight.numel() != experts * bytes_per_expert:
        _fail("packed_weight byte count is inconsistent with its grouped physical shape")
    _check_aligned(activation, name)
    _check_aligned(packed_weight, "packed_weight")
    return rows, in_features, out_features, experts, groups, bytes_per_expert


def same_weight_geometry(first: torch.Tensor, second: torch.Tensor) -> bool:
    """Whether ``second`` would pass every check that ``first`` has passed as a call's packed weight: same dtype, device
    and shape, contiguous from the start of its storage, 16-byte aligned.  A pair's second weight that does is not
    checked a second time (decode-sized calls spend a fifth of their host time there); one that does not goes
    through ``grouped`` for that function's message."""
    return (
        second.dtype == first.dtype and second.device == first.device and second.shape == first.shape
        and second.is_contiguous() and second.storage_offset() == 0 and second.data_ptr() % 16 == 0
    )


def activation(tensor: torch.Tensor, name: str) -> None:
    """Checks of a bf16 activation tensor that is quantized on its own (quantize_q8_1)."""
    _check_tensor(tensor, name, torch.bfloat16, "torch.bfloat16")
    _check_layout(tensor, name)
    if tensor.dim() < 1:
        _fail(f"{name} must have at least one dimension")
    in_features = int(tensor.shape[-1])
    if in_features <= 0 or in_features % QK_K != 0:
        _fail(f"{name} width must be a positive multiple of 256; got {in_features}")
    rows = tensor.numel() // in_features
    if rows <= 0:
        _fail(f"zero-row {name} tensors are not supported")
    if rows > _INT_MAX:
        _fail(f"flattened {name} row count exceeds the kernel limit")
    _check_aligned(tensor, name)


def prepared(
    workspace: torch.Tensor, packed_weight: torch.Tensor, rows: int, in_features: int, quant_type: int, out_features: int
) -> None:
    """Checks of mmq_prepared: a q8_1 workspace instead of an activation tensor, otherwise as for mmq."""
    _check_tensor(workspace, "workspace", torch.uint8, "torch.uint8")
    _check_tensor(packed_weight, "packed_weight", torch.uint8, "torch.uint8")
    if workspace.device != packed_weight.device:
        _fail("workspace and packed_weight must be on the same device")
    _check_layout(workspace, "workspace")
    _check_layout(packed_weight, "packed_weight")
    if in_features <= 0 or in_features % QK_K != 0:
        _fail(f"input width must be a positive multiple of 256; got {in_features}")
    if out_features <= 0:
        _fail(f"out_features must be positive; got {out_features}")
    if rows <= 0:
        _fail("zero-row inputs are not supported")
    if rows > _INT_MAX or in_features > _INT_MAX or out_features > _INT_MAX:
        _fail("shape exceeds the kernel limit")
    expected = out_features * (in_features // QK_K) * packed_block_bytes(quant_type)
    if packed_weight.numel() != expected:
        _fail(
            f"packed_weight has {packed_weight.numel()} bytes, expected {expected} for "
            f"[{out_features}, {in_features}] quant_type={quant_type}"
        )
    _check_aligned(workspace, "workspace")
    _check_aligned(packed_weight, "packed_weight")


def row_index(index: torch.Tensor, activation: torch.Tensor) -> int:
    """Checks the token -> sorted-row gather index of the gathered grouped operators.  Returns its length."""
    if REQUIRE_DEVICE and not index.is_cuda:
        _fail("row_index must be a CUDA/HIP tensor")
    if index.device != activation.device:
        _fail("all grouped MMQ tensors must be on the same device")
    if index.dtype != torch.int64:
        _fail("row_index must have dtype torch.int64")
    if index.dim() != 1:
        _fail("row_index must be one-dimensional")
    if not index.is_contiguous():
        _fail("row_index must be contiguous; torch_ggml_ops will not insert a hidden copy")
    if index.numel() <= 0:
        _fail("zero-row inputs are not supported")
    return int(index.numel())
