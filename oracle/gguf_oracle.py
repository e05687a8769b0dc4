"""ctypes front end of the CPU oracle (libgguf_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the CPU-baseline leg of the benchmark may
import this module; the shipped operators never do.  bf16 data crosses this
boundary as numpy ``uint16`` bit patterns, packed GGUF rows as ``uint8``.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "libgguf_oracle.so"

Q3_K, Q4_K, Q5_K, Q6_K, IQ2_S = 11, 12, 13, 14, 22
QUANT_TYPES = {"Q3_K": Q3_K, "Q4_K": Q4_K, "Q5_K": Q5_K, "Q6_K": Q6_K, "IQ2_S": IQ2_S}
BLOCK_BYTES = {Q3_K: 110, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ2_S: 82}


def build(force: bool = False) -> Path:
    """Compile the oracle with gcc through its Makefile."""
    if force or not _LIB_PATH.exists():
        if force:
            subprocess.run(["make", "-C", str(_DIR), "clean"], check=True, capture_output=True)
        subprocess.run(["make", "-C", str(_DIR)], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
        i64, p = ctypes.c_int64, ctypes.c_void_p
        _lib.tgo_oracle_block_bytes.argtypes = [ctypes.c_int]
        _lib.tgo_oracle_block_bytes.restype = ctypes.c_int
        _lib.tgo_oracle_iq2s_grid.argtypes = [p]
        _lib.tgo_oracle_decode_value.argtypes = [ctypes.c_int, p, ctypes.c_int, ctypes.c_int]
        _lib.tgo_oracle_decode_value.restype = ctypes.c_float
        _lib.tgo_oracle_dequant_f32.argtypes = [ctypes.c_int, p, i64, i64, p]
        _lib.tgo_oracle_dequant_bf16.argtypes = [ctypes.c_int, p, i64, i64, p]
        _lib.tgo_oracle_f32_to_bf16.argtypes = [p, i64, p]
        _lib.tgo_oracle_quantize_q8_1.argtypes = [p, i64, i64, p, p, p]
        _lib.tgo_oracle_round_to_half.argtypes = [p, i64, p]
        for name in ("tgo_oracle_mmq_forward", "tgo_oracle_mmq_forward_half_scales", "tgo_oracle_linear_forward",
                     "tgo_oracle_grad_input"):
            getattr(_lib, name).argtypes = [ctypes.c_int, p, p, i64, i64, i64, p]
    return _lib


def _ptr(array: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(array.ctypes.data)


def _c(array: np.ndarray, dtype) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=dtype)


def row_bytes(qtype: int, in_features: int) -> int:
    return (in_features // 256) * BLOCK_BYTES[qtype]


def iq2s_grid() -> np.ndarray:
    out = np.empty(1024, dtype=np.uint64)
    lib().tgo_oracle_iq2s_grid(_ptr(out))
    return out


def decode_value(qtype: int, packed_row: np.ndarray, block_index: int, value_index: int) -> float:
    packed_row = _c(packed_row, np.uint8)
    return float(lib().tgo_oracle_decode_value(qtype, _ptr(packed_row), block_index, value_index))


def dequant_f32(qtype: int, packed: np.ndarray, in_features: int) -> np.ndarray:
    """packed uint8 [..., row_bytes] -> float32 [..., in_features]."""
    packed = _c(packed, np.uint8)
    rows = packed.size // row_bytes(qtype, in_features)
    out = np.empty((rows, in_features), dtype=np.float32)
    lib().tgo_oracle_dequant_f32(qtype, _ptr(packed), rows, in_features, _ptr(out))
    return out.reshape(*packed.shape[:-1], in_features)


def dequant_bf16(qtype: int, packed: np.ndarray, in_features: int) -> np.ndarray:
    """packed uint8 [..., row_bytes] -> bf16 bit patterns uint16 [..., in_features]."""
    packed = _c(packed, np.uint8)
    rows = packed.size // row_bytes(qtype, in_features)
    out = np.empty((rows, in_features), dtype=np.uint16)
    lib().tgo_oracle_dequant_bf16(qtype, _ptr(packed), rows, in_features, _ptr(out))
    return out.reshape(*packed.shape[:-1], in_features)


def f32_to_bf16(values: np.ndarray) -> np.ndarray:
    values = _c(values, np.float32)
    out = np.empty(values.shape, dtype=np.uint16)
    lib().tgo_oracle_f32_to_bf16(_ptr(values), values.size, _ptr(out))
    return out


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def quantize_q8_1(x_bf16: np.ndarray):
    """bf16 bits [rows, K] -> (int8 [rows, K], d float32 [rows, K/32], sum float32 [rows, K/32])."""
    x_bf16 = _c(x_bf16, np.uint16)
    rows, k = x_bf16.shape
    q = np.empty((rows, k), dtype=np.int8)
    d = np.empty((rows, k // 32), dtype=np.float32)
    s = np.empty((rows, k // 32), dtype=np.float32)
    lib().tgo_oracle_quantize_q8_1(_ptr(x_bf16), rows, k, _ptr(q), _ptr(d), _ptr(s))
    return q, d, s


def _matmul(name: str, qtype: int, lhs_bf16: np.ndarray, packed: np.ndarray,
            out_features: int, in_features: int, out_cols: int) -> np.ndarray:
    lhs_bf16 = _c(lhs_bf16, np.uint16)
    packed = _c(packed, np.uint8)
    rows = lhs_bf16.shape[0]
    assert packed.size == out_features * row_bytes(qtype, in_features)
    out = np.empty((rows, out_cols), dtype=np.float32)
    getattr(lib(), name)(qtype, _ptr(lhs_bf16), _ptr(packed), rows, out_features, in_features, _ptr(out))
    return out


def mmq_forward(qtype, x_bf16, packed, out_features, in_features) -> np.ndarray:
    """Quantized-activation forward algebra, float64 accumulation -> float32 [rows, N]."""
    assert x_bf16.shape[1] == in_features
    return _matmul("tgo_oracle_mmq_forward", qtype, x_bf16, packed, out_features, in_features, out_features)


def mmq_forward_half_scales(qtype, x_bf16, packed, out_features, in_features) -> np.ndarray:
    """mmq_forward with the per-block scale values of Q4_K / Q5_K rounded to fp16 where the reference keeps them
    as half2 (weights: d*sc and -dmin*m; activations: d and sum); other formats: identical to mmq_forward."""
    assert x_bf16.shape[1] == in_features
    return _matmul("tgo_oracle_mmq_forward_half_scales", qtype, x_bf16, packed, out_features, in_features, out_features)


def round_to_half(values: np.ndarray) -> np.ndarray:
    """float32 -> nearest fp16 value (ties to even), returned as float32."""
    values = _c(values, np.float32)
    out = np.empty_like(values)
    lib().tgo_oracle_round_to_half(_ptr(values), values.size, _ptr(out))
    return out


def linear_forward(qtype, x_bf16, packed, out_features, in_features) -> np.ndarray:
    """x @ bf16(W)^T, float64 accumulation -> float32 [rows, N]."""
    assert x_bf16.shape[1] == in_features
    return _matmul("tgo_oracle_linear_forward", qtype, x_bf16, packed, out_features, in_features, out_features)


def grad_input(qtype, dy_bf16, packed, out_features, in_features) -> np.ndarray:
    """dY @ bf16(W), float64 accumulation -> float32 [rows, K]."""
    assert dy_bf16.shape[1] == out_features
    return _matmul("tgo_oracle_grad_input", qtype, dy_bf16, packed, out_features, in_features, in_features)


def grouped(fn, qtype, lhs_bf16, packed_experts, expert_indices, expert_offsets,
            out_features, in_features, out_cols) -> np.ndarray:
    """Apply a dense oracle function per expert group of expert-sorted rows.

    Rows outside every valid group stay NaN: the operators leave them
    uninitialised (reference: csrc/mmq_core.cuh:466-476 skips invalid groups).
    """
    rows = lhs_bf16.shape[0]
    out = np.full((rows, out_cols), np.nan, dtype=np.float32)
    begin = 0
    for expert, end in zip(np.asarray(expert_indices).tolist(), np.asarray(expert_offsets).tolist()):
        valid = 0 <= expert < packed_experts.shape[0] and begin >= 0 and end > begin and end <= rows
        if valid:
            out[begin:end] = fn(qtype, lhs_bf16[begin:end], packed_experts[expert], out_features, in_features)
        begin = end
    return out
