"""Arithmetic facts the fp16-operand forward kernels rely on, checked exhaustively on the CPU.

The kernels multiply fp16 numbers that are meant to hold integers exactly (quantized activations and
`sub-scale x quant` weight operands) and read the block dot product out of the matrix instruction's fp32
accumulator.  That is exact when (a) every operand value is representable in fp16, (b) every product is
representable in fp32 and (c) the absolute values of a 32-value block's products add up to less than 2^24,
so that no partial sum, in whatever order the hardware adds, needs rounding.  The unpackers form the operands
with fp16 arithmetic on `1024 + byte` (the byte placed under the bits of 1024.0); those steps are restated here
with numpy's float16, which rounds every operation, so an inexact step would show.
"""

import numpy as np

MAX_ACTIVATION = 127          # |q8_1 quant|
BLOCK = 32                    # values per q8_1 block = per chained group of matrix instructions
LIMIT = 2**24


def _exact_in_half(values):
    values = np.asarray(values, dtype=np.float64)
    with np.errstate(over="ignore"):   # (a value beyond the fp16 range becomes infinity, which is "not exact")
        return np.array_equal(values.astype(np.float16).astype(np.float64), values)


def _operand_sets():
    """(name, weight operand values per fp16 number) for every format, over all sub-scales and quants."""
    sets = {}
    sc = np.arange(64)                                             # 6-bit scale of Q4_K / Q5_K
    sets["Q4_K"] = [np.multiply.outer(sc, np.arange(16)).ravel()]
    sets["Q5_K"] = [np.multiply.outer(sc, np.arange(32)).ravel()]
    sets["Q3_K"] = [np.multiply.outer(np.arange(-32, 32), np.arange(-4, 4)).ravel()]
    signed = np.concatenate([m * np.array([-1, 1]) for m in (8, 25, 43)])
    sets["IQ2_S"] = [np.multiply.outer(2 * np.arange(16) + 1, signed).ravel()]
    sc6 = np.arange(-128, 128)
    magnitude = np.abs(sc6)
    coarse = np.sign(sc6) * (magnitude & ~15)
    fine = np.sign(sc6) * (magnitude & 15)
    assert np.array_equal(coarse + fine, sc6)
    assert np.array_equal(np.abs(coarse) + np.abs(fine), magnitude)   # both parts carry the sign of the scale
    q6 = np.arange(-32, 32)
    sets["Q6_K"] = [np.multiply.outer(coarse, q6).ravel(), np.multiply.outer(fine, q6).ravel()]
    return sets


def test_every_operand_value_is_a_half():
    assert _exact_in_half(np.arange(-MAX_ACTIVATION, MAX_ACTIVATION + 1))
    for name, planes in _operand_sets().items():
        for values in planes:
            assert _exact_in_half(values), name


def test_block_sums_stay_below_two_to_the_24():
    """Sum of |activation| * |operand| over a block, all numbers of a value counted (Q6_K has two)."""
    for name, planes in _operand_sets().items():
        worst = sum(int(np.abs(values).max()) for values in planes) if name != "Q6_K" else 128 * 32
        assert BLOCK * MAX_ACTIVATION * worst < LIMIT, name
    # Q6_K with the split taken by value instead of by magnitude (fine part 0..15 for negative scales as well)
    # would break the bound: the parts of scale -113 are -128 and +15, 143 in absolute value
    assert BLOCK * MAX_ACTIVATION * 32 * (128 + 15) >= LIMIT


def test_unpack_steps_are_exact_in_half_precision():
    half = np.float16
    bias = half(1024.0)
    # byte under the bits of 1024.0 is the number 1024 + byte
    bytes_ = np.arange(256, dtype=np.uint16)
    assert np.array_equal((np.uint16(0x6400) | bytes_).view(np.float16).astype(np.float64), 1024.0 + bytes_)
    # fma(1024 + b, m, -1024 m) = b * m (Q4_K / Q5_K / IQ2_S): the product is formed exactly inside the fma, so only
    # the operands and the result have to be halves
    for quants, multipliers in ((np.arange(32), np.arange(64)), (np.array([8, 25, 43]), 2 * np.arange(16) + 1)):
        assert _exact_in_half(-1024.0 * multipliers)
        assert _exact_in_half(np.multiply.outer(quants, multipliers))
    # Q3_K and Q6_K subtract first and multiply after: both steps rounded by numpy, both exact
    for offset, quants, multipliers in ((4, np.arange(8), np.arange(-32, 32)), (32, np.arange(64), np.arange(-128, 128, 1))):
        centred = (bias + quants.astype(half)) - half(1024 + offset)
        assert np.array_equal(centred.astype(np.float64), quants - offset)
        usable = multipliers if offset == 4 else np.unique(np.concatenate(
            [np.sign(multipliers) * (np.abs(multipliers) & ~15), np.sign(multipliers) * (np.abs(multipliers) & 15)]))
        products = np.multiply.outer(centred, usable.astype(half))
        assert products.dtype == np.float16
        assert np.array_equal(products.astype(np.float64), np.multiply.outer(quants - offset, usable))
    # the single-step form would not do for them: (1024 + offset) * multiplier is not always a half
    assert not _exact_in_half(1028.0 * np.arange(-32, 32))
    assert not _exact_in_half(1056.0 * 16.0 * np.arange(-8, 8))   # and overflows for the larger scales


def test_quantizer_forms_the_activation_halves_exactly():
    magnitudes = np.arange(128, dtype=np.uint16)
    halves = (np.uint16(0x6400) | magnitudes).view(np.float16) - np.float16(1024.0)
    assert np.array_equal(halves.astype(np.float64), magnitudes)
    negative = (halves.view(np.uint16) | np.uint16(0x8000)).view(np.float16)   # the sign bit copied from the input
    assert np.array_equal(negative.astype(np.float64)[1:], -magnitudes[1:].astype(np.float64))
