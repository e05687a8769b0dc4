"""Conversion and comparison helpers shared by the GPU parity tests."""

import numpy as np
import torch

QTYPES = {"Q3_K": 11, "Q4_K": 12, "Q5_K": 13, "Q6_K": 14, "IQ2_S": 22}


def bits(tensor: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> numpy uint16 bit patterns (host)."""
    return tensor.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def from_bits(array: np.ndarray, device="cuda") -> torch.Tensor:
    return torch.from_numpy(array.view(np.int16).copy()).view(torch.bfloat16).to(device)


def f32(tensor: torch.Tensor) -> np.ndarray:
    return tensor.detach().float().cpu().numpy()


def nrmse(actual: np.ndarray, expected: np.ndarray) -> float:
    actual = actual.astype(np.float64)
    expected = expected.astype(np.float64)
    return float(np.sqrt(np.mean((actual - expected) ** 2)) / np.sqrt(np.mean(expected**2)))


def max_rel_to_peak(actual: np.ndarray, expected: np.ndarray) -> float:
    """max |error| / max |reference|: the norm-relative reading of 'max relative error'."""
    return float(np.abs(actual.astype(np.float64) - expected).max() / np.abs(expected).max())


def assert_matches_f32_reference(actual_bf16: torch.Tensor, reference_f32: np.ndarray, accumulate_noise=1e-4):
    """A bf16 result equals a float32 reference up to its own rounding (2^-8 relative, i.e. one
    ulp) plus fp32 accumulation noise measured against the largest reference magnitude."""
    actual = f32(actual_bf16).astype(np.float64)
    reference = reference_f32.astype(np.float64)
    tolerance = np.abs(reference) * 2.0**-8 + accumulate_noise * np.abs(reference).max()
    error = np.abs(actual - reference)
    worst = np.unravel_index(np.argmax(error - tolerance), error.shape)
    assert (error <= tolerance).all(), (
        f"worst at {worst}: got {actual[worst]}, reference {reference[worst]}, "
        f"error {error[worst]:.3e} > tolerance {tolerance[worst]:.3e}"
    )


# Noise allowance of assert_matches_f32_reference by operand kind of the forward kernel.  int8 and exact fp16 operands
# compute the oracle's integer dot products and differ from it by fp32 summation order only.  The scaled kind rounds
# every dequantized activation and weight to fp16 once (2^-11 relative each): with random signs the dot product's
# error is a few 1e-4 of the largest output (measured: up to 2.9e-4 at K of 256 to 4096, up to 4.6e-4 for Q4_K/Q5_K at
# 4096 rows, whose minimum term cancels a large part of the sum).
OPERAND_NOISE = {"int8": 1e-4, "half": 1e-4, "scaled": 8e-4}


def forward_noise(qtype: int, rows: int, out_features: int, projections: int = 1) -> float:
    """Allowance for the kind the library uses for a forward call of this shape under the current setting (total rows
    of a grouped call; projections: 2 for a pair)."""
    from torch_ggml_ops import _native

    return OPERAND_NOISE[_native.forward_operand_for(qtype, rows, out_features, projections)]


def random_bf16(shape, seed, device="cuda", scale=1.0) -> torch.Tensor:
    generator = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=generator) * scale).to(torch.bfloat16).to(device)
