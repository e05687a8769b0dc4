"""ctypes binding of libtgo_hip.so (the C ABI declared in include/tgo.h).

The library is built in-tree by ``torch-ggml-ops_amd/csrc/Makefile``.  There is no
fallback: if it is missing, importing the package fails.
"""

from __future__ import annotations

import contextlib
import ctypes
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent / "libtgo_hip.so"

if not _LIB_PATH.exists():
    raise ImportError(
        f"{_LIB_PATH} is missing: build it with `make -C torch-ggml-ops_amd/csrc` "
        "(torch_ggml_ops has no fallback path without its HIP library)"
    )

lib = ctypes.CDLL(str(_LIB_PATH))

_p, _i64, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

lib.tgo_version.restype = _int
lib.tgo_last_error.restype = ctypes.c_char_p
lib.tgo_block_bytes.argtypes = [_int]
lib.tgo_block_bytes.restype = _int
lib.tgo_q8_workspace_bytes.argtypes = [_i64, _i64]
lib.tgo_q8_workspace_bytes.restype = _i64
lib.tgo_task_workspace_bytes.argtypes = [_i64, _i64]
lib.tgo_task_workspace_bytes.restype = _i64
lib.tgo_forward_kernel_family.argtypes = [_i64, _i64]
lib.tgo_forward_kernel_family.restype = ctypes.c_char_p
lib.tgo_dequant_bf16.argtypes = [_p, _p, _i64, _i64, _int, _p]
lib.tgo_quantize_q8_1.argtypes = [_p, _p, _i64, _i64, _p]
lib.tgo_q8_workspace_unpack.argtypes = [_p, _p, _p, _p, _i64, _i64, _p]
lib.tgo_mmq_forward.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _p]
lib.tgo_mmq_forward_static.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _p]
lib.tgo_mmq_forward_prepared.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _p]
lib.tgo_quantize_q8_1_as.argtypes = [_p, _p, _i64, _i64, _int, _p]
lib.tgo_mmq_forward_prepared_as.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _int, _p]
lib.tgo_grad_workspace_bytes.argtypes = [_i64, _i64, _i64, _int]
lib.tgo_grad_workspace_bytes.restype = _i64
lib.tgo_dense_grad_workspace_bytes.argtypes = [_i64, _i64, _i64, _int]
lib.tgo_dense_grad_workspace_bytes.restype = _i64
lib.tgo_mmq_grad_input.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _int, _p]
lib.tgo_grouped_mmq_forward.argtypes = [_p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int, _p]
lib.tgo_grouped_mmq_forward_gathered.argtypes = [_p, _p, _i64, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int, _p]
lib.tgo_grouped_mmq_swiglu.argtypes = [_p, _p, _i64, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int, _p]
lib.tgo_swiglu_rows.argtypes = [_p, _p, _p, _i64, _p]
lib.tgo_swiglu_backward.argtypes = [_p, _p, _p, _p, _p, _p, _i64, _p]
lib.tgo_route_small.argtypes = [_p, _i64, _i64, _i64, _p, _p, _p, _p, _p]
lib.tgo_rows_to_tokens.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _p]
lib.tgo_moe_combine.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _p]
lib.tgo_grouped_mmq_grad_input.argtypes = [_p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int, _p]
lib.tgo_grouped_mmq_grad_input_weighted.argtypes = [_p, _p, _p, _i64, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _int, _p]
lib.tgo_profile_enable.argtypes = [_int]
lib.tgo_profile_read.argtypes = [_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int64)]
lib.tgo_set_forward_operand.argtypes = [_int]
lib.tgo_forward_operand.argtypes = []
lib.tgo_forward_operand_for.argtypes = [_int, _i64, _i64, _int]

KERNEL_IDS = {
    "quantize": 0, "build_tasks": 1, "forward": 2, "grad_input": 3, "dequant": 4, "forward_gemv": 5,
    "pack_cotangent": 6, "combine": 7,
}

EXPORTS = (
    "tgo_version",
    "tgo_dense_grad_workspace_bytes",
    "tgo_grad_workspace_bytes",
    "tgo_last_error",
    "tgo_block_bytes",
    "tgo_q8_workspace_bytes",
    "tgo_task_workspace_bytes",
    "tgo_forward_kernel_family",
    "tgo_dequant_bf16",
    "tgo_quantize_q8_1",
    "tgo_q8_workspace_unpack",
    "tgo_mmq_forward",
    "tgo_mmq_forward_static",
    "tgo_mmq_forward_prepared",
    "tgo_quantize_q8_1_as",
    "tgo_mmq_forward_prepared_as",
    "tgo_mmq_grad_input",
    "tgo_grouped_mmq_forward",
    "tgo_grouped_mmq_forward_gathered",
    "tgo_grouped_mmq_swiglu",
    "tgo_swiglu_rows",
    "tgo_swiglu_backward",
    "tgo_route_small",
    "tgo_rows_to_tokens",
    "tgo_moe_combine",
    "tgo_grouped_mmq_grad_input",
    "tgo_grouped_mmq_grad_input_weighted",
    "tgo_profile_enable",
    "tgo_profile_read",
    "tgo_set_forward_operand",
    "tgo_forward_operand",
    "tgo_forward_operand_for",
)

OPERANDS = {"int8": 0, "half": 1, "auto": 2, "scaled": 3}


def set_forward_operand(operand: str) -> None:
    """Matrix operands of the MFMA forward kernels: "int8", "half" (fp16 numbers holding the exact integers),
    "scaled" (dequantized activations and weights as fp16, normalised per row: the kind bounded by the matrix
    pipe), or "auto" (the default: scaled for calls that fill the chip, otherwise half for IQ2_S and int8 for
    the other formats)."""
    check(lib.tgo_set_forward_operand(OPERANDS[operand]))


def forward_operand() -> str:
    return {value: name for name, value in OPERANDS.items()}[lib.tgo_forward_operand()]


def forward_operand_for(quant_type: int, rows: int, out_features: int, projections: int = 1) -> str:
    """The kind a forward call of this format and shape uses under the current setting (never "auto")."""
    return {value: name for name, value in OPERANDS.items()}[lib.tgo_forward_operand_for(quant_type, rows, out_features, projections)]


def profile_read(kernel: str) -> tuple[float, int]:
    """(summed milliseconds, launches) of one kernel since tgo_profile_enable(1)."""
    total, count = ctypes.c_double(0.0), ctypes.c_int64(0)
    check(lib.tgo_profile_read(KERNEL_IDS[kernel], ctypes.byref(total), ctypes.byref(count)))
    return total.value, count.value


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)
_STAY = contextlib.nullcontext()


def stream_of(device: torch.device) -> int:
    """Handle of torch's current stream on ``device``, the value of ``torch.cuda.current_stream(device).cuda_stream``:
    taken through torch's raw call where it has one, because building the Stream object costs a decode-sized call a
    quarter of its host time."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def on_device(device: torch.device):
    """Context in which ``device`` is the current device; nothing is entered when it already is."""
    if _current_device is not None and device.index is not None and _current_device() == device.index:
        return _STAY
    return torch.cuda.device(device)


def check(status: int) -> None:
    """Raise the library's message as RuntimeError when a call reports failure."""
    if status != 0:
        raise RuntimeError(lib.tgo_last_error().decode())
