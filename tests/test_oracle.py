"""Pins the CPU oracle before anything is compared against it (CPU only).

The reference ships no golden vectors (its tests read an external checkpoint), so
the oracle is pinned by what the formats and the mathematics fix:
  * blocks *encoded* here from chosen integer fields, whose decoded values are known
    in closed form (an encoder exercises the inverse index/shift arithmetic);
  * an independent numpy decoder following ggml's row dequantizers;
  * the IQ2_S codebook's checksum and the two entries the reference's file shows
    first and last;
  * invariants of the q8_1 quantizer and brute force on its rounding;
  * float64 numpy matmuls for the three matmul helpers.
"""

import hashlib
import json
from pathlib import Path

import numpy as np
import pytest

import npdecode

GOLDEN = Path(__file__).parent / "golden"
Q3_K, Q4_K, Q5_K, Q6_K, IQ2_S = 11, 12, 13, 14, 22
ALL_TYPES = [Q3_K, Q4_K, Q5_K, Q6_K, IQ2_S]


def _half_bytes(value: float) -> np.ndarray:
    return np.frombuffer(np.float16(value).tobytes(), dtype=np.uint8)


def _bf16_bits(values: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bits, round to nearest even (independent of the oracle)."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    return rounded.astype(np.uint16)


def _bf16_round(values: np.ndarray) -> np.ndarray:
    return (_bf16_bits(values).astype(np.uint32) << 16).view(np.float32)


# ---- encoders: integer fields -> packed block ------------------------------------


def _encode_k_scales(sc, mn) -> np.ndarray:
    """Eight 6-bit scales and mins -> the 12-byte field of Q4_K/Q5_K."""
    out = np.zeros(12, dtype=np.uint8)
    for j in range(8):
        if j < 4:
            out[j] |= sc[j] & 63
            out[j + 4] |= mn[j] & 63
        else:
            out[j + 4] = (sc[j] & 0x0F) | ((mn[j] & 0x0F) << 4)
            out[j - 4] |= (sc[j] >> 4) << 6
            out[j] |= (mn[j] >> 4) << 6
    return out


def encode_q4_k(d, dmin, sc, mn, q) -> np.ndarray:
    block = np.zeros(144, dtype=np.uint8)
    block[0:2], block[2:4] = _half_bytes(d), _half_bytes(dmin)
    block[4:16] = _encode_k_scales(sc, mn)
    for i in range(256):
        group = i // 32
        byte = 16 + (group // 2) * 32 + i % 32
        block[byte] |= (q[i] & 0x0F) << (4 * (group % 2))
    return block


def encode_q5_k(d, dmin, sc, mn, q) -> np.ndarray:
    block = np.zeros(176, dtype=np.uint8)
    block[0:2], block[2:4] = _half_bytes(d), _half_bytes(dmin)
    block[4:16] = _encode_k_scales(sc, mn)
    for i in range(256):
        group = i // 32
        block[48 + (group // 2) * 32 + i % 32] |= (q[i] & 0x0F) << (4 * (group % 2))
        block[16 + i % 32] |= ((q[i] >> 4) & 1) << group
    return block


def encode_q6_k(d, sc, q) -> np.ndarray:
    """q in [-32, 31], sc int8 per 16 values."""
    block = np.zeros(210, dtype=np.uint8)
    for i in range(256):
        u = q[i] + 32
        chunk, rem = i // 128, i % 128
        block[chunk * 64 + rem % 64] |= (u & 0x0F) << (4 * (rem // 64))
        block[128 + chunk * 32 + i % 32] |= (u >> 4) << (2 * (rem // 32))
    block[192:208] = np.array(sc, dtype=np.int8).view(np.uint8)
    block[208:210] = _half_bytes(d)
    return block


def encode_q3_k(d, sc, q) -> np.ndarray:
    """q in [-4, 3], sc in [-32, 31] per 16 values."""
    block = np.zeros(110, dtype=np.uint8)
    for i in range(256):
        u = q[i] + 4
        chunk, rem = i // 128, i % 128
        block[32 + chunk * 32 + rem % 32] |= (u & 3) << (2 * (rem // 32))
        block[i % 32] |= (u >> 2) << (i // 32)
    for group in range(16):
        u = sc[group] + 32
        if group < 8:
            block[96 + group] |= u & 0x0F
        else:
            block[96 + group - 8] |= (u & 0x0F) << 4
        block[96 + 8 + group % 4] |= (u >> 4) << (2 * (group // 4))
    block[108:110] = _half_bytes(d)
    return block


def encode_iq2_s(d, grid_index, negative, scale4) -> np.ndarray:
    """32 grid indices (10 bit), 256 sign flags, 16 four-bit scales."""
    block = np.zeros(82, dtype=np.uint8)
    block[0:2] = _half_bytes(d)
    for group in range(32):
        block[2 + group] = grid_index[group] & 0xFF
        block[66 + group // 4] |= (grid_index[group] >> 8) << (2 * (group % 4))
        for e in range(8):
            block[34 + group] |= int(negative[group * 8 + e]) << e
    for sub in range(16):
        block[74 + sub // 2] |= (scale4[sub] & 0x0F) << (4 * (sub % 2))
    return block


# ---- codebook --------------------------------------------------------------------


def test_codebook_matches_reference_table(oracle):
    grid = oracle.iq2s_grid()
    golden = json.loads((GOLDEN / "iq2s_grid.json").read_text())
    assert grid[0] == 0x0808080808080808
    assert grid[1] == 0x080808080808082B
    assert grid[2] == 0x0808080808081919
    assert grid[1023] == 0x2B2B2B2B2B2B2B2B
    assert hashlib.sha256(grid.astype("<u8").tobytes()).hexdigest() == golden["sha256_le_u64"]
    assert int(grid.sum(dtype=np.uint64)) == golden["sum_mod_2_64"]
    assert set(np.unique(grid.view(np.uint8)).tolist()) == {0x08, 0x19, 0x2B}


# ---- known-answer blocks -----------------------------------------------------------


def test_q4_k_known_answer(oracle):
    sc = [1, 2, 3, 4, 37, 48, 59, 63]
    mn = [0, 5, 10, 15, 33, 44, 55, 62]
    q = [(7 * i + 3) % 16 for i in range(256)]
    block = encode_q4_k(2.0, 0.5, sc, mn, q)
    expected = np.array([2.0 * sc[i // 32] * q[i] - 0.5 * mn[i // 32] for i in range(256)], dtype=np.float32)
    np.testing.assert_array_equal(oracle.dequant_f32(Q4_K, block[None], 256)[0], expected)


def test_q5_k_known_answer(oracle):
    sc = [63, 1, 17, 32, 16, 47, 5, 60]
    mn = [9, 0, 63, 31, 48, 16, 1, 35]
    q = [(11 * i + 5) % 32 for i in range(256)]
    block = encode_q5_k(0.25, 4.0, sc, mn, q)
    expected = np.array([0.25 * sc[i // 32] * q[i] - 4.0 * mn[i // 32] for i in range(256)], dtype=np.float32)
    np.testing.assert_array_equal(oracle.dequant_f32(Q5_K, block[None], 256)[0], expected)


def test_q6_k_known_answer(oracle):
    sc = [-128, 127, 1, -1, 5, -7, 64, -64, 33, 2, -3, 100, -100, 17, 0, 9]
    q = [((13 * i + 7) % 64) - 32 for i in range(256)]
    block = encode_q6_k(0.5, sc, q)
    expected = np.array([0.5 * sc[i // 16] * q[i] for i in range(256)], dtype=np.float32)
    np.testing.assert_array_equal(oracle.dequant_f32(Q6_K, block[None], 256)[0], expected)


def test_q3_k_known_answer(oracle):
    sc = [-32, 31, 0, 1, -1, 15, -16, 7, 20, -20, 3, -3, 30, -31, 8, -8]
    q = [((5 * i + 2) % 8) - 4 for i in range(256)]
    block = encode_q3_k(3.0, sc, q)
    expected = np.array([3.0 * sc[i // 16] * q[i] for i in range(256)], dtype=np.float32)
    np.testing.assert_array_equal(oracle.dequant_f32(Q3_K, block[None], 256)[0], expected)


def test_iq2_s_known_answer(oracle):
    grid = oracle.iq2s_grid().astype("<u8").view(np.uint8).reshape(1024, 8)
    rng = np.random.default_rng(7)
    index = [0, 1023, 1, 512, 255, 256, 767, 768] + rng.integers(0, 1024, 24).tolist()
    negative = rng.integers(0, 2, 256)
    scale4 = list(range(16))
    block = encode_iq2_s(8.0, index, negative, scale4)
    expected = np.zeros(256, dtype=np.float32)
    for i in range(256):
        magnitude = float(grid[index[i // 8], i % 8])
        expected[i] = 8.0 * (0.5 + scale4[i // 16]) * 0.25 * magnitude * (-1.0 if negative[i] else 1.0)
    np.testing.assert_array_equal(oracle.dequant_f32(IQ2_S, block[None], 256)[0], expected)


def test_single_value_accessor_agrees_with_row_decoder(oracle):
    rng = np.random.default_rng(3)
    for qtype in ALL_TYPES:
        row = _random_rows(rng, qtype, 1, 512)
        full = oracle.dequant_f32(qtype, row, 512)[0]
        for position in (0, 1, 15, 16, 31, 32, 127, 128, 255, 256, 300, 511):
            assert oracle.decode_value(qtype, row[0], position // 256, position % 256) == full[position]


# ---- independent decoder on random blocks ------------------------------------------


def _random_rows(rng, qtype, rows, in_features, subnormal_scales=False):
    import synth

    block = synth.BLOCK_BYTES[qtype]
    count = rows * (in_features // 256)
    data = rng.integers(0, 256, (count, block), dtype=np.uint8)
    for offset in synth._SCALE_FIELDS[qtype]:
        if subnormal_scales:
            raw = rng.integers(1, 0x0400, count).astype(np.uint16) | (rng.integers(0, 2, count).astype(np.uint16) << 15)
        else:
            # any finite fp16, both signs: exponent field 1..30
            raw = (
                (rng.integers(0, 2, count).astype(np.uint16) << 15)
                | (rng.integers(1, 31, count).astype(np.uint16) << 10)
                | rng.integers(0, 1024, count).astype(np.uint16)
            )
        data[:, offset : offset + 2] = raw.view(np.uint8).reshape(count, 2)
    return data.reshape(rows, -1)


@pytest.mark.parametrize("qtype", ALL_TYPES)
@pytest.mark.parametrize("subnormal", [False, True])
def test_dequant_agrees_with_independent_decoder(oracle, qtype, subnormal):
    rng = np.random.default_rng(1000 + qtype)
    packed = _random_rows(rng, qtype, 6, 512, subnormal_scales=subnormal)
    expected = npdecode.dequant_rows(qtype, packed, 512, oracle.iq2s_grid())
    actual = oracle.dequant_f32(qtype, packed, 512)
    np.testing.assert_array_equal(actual.view(np.uint32), expected.view(np.uint32))
    np.testing.assert_array_equal(oracle.dequant_bf16(qtype, packed, 512), _bf16_bits(expected))


def test_bf16_rounding_is_nearest_even(oracle):
    values = np.array(
        [1.0, 1.00390625, 1.005859375, 1.01171875, -1.00390625, 3.3895314e38, 1e-40, 0.0, -0.0],
        dtype=np.float32,
    )
    # 1 + 2^-8 is a tie -> even (1.0); 1 + 3*2^-9 rounds up; 1 + 3*2^-8 is a tie -> up to even
    expected = np.array([0x3F80, 0x3F80, 0x3F81, 0x3F82, 0xBF80, 0x7F7F, 0x0001, 0x0000, 0x8000], dtype=np.uint16)
    np.testing.assert_array_equal(oracle.f32_to_bf16(values), expected)
    rng = np.random.default_rng(0)
    many = rng.standard_normal(4096).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 4096)
    np.testing.assert_array_equal(oracle.f32_to_bf16(many), _bf16_bits(many.astype(np.float32)))


# ---- q8_1 ----------------------------------------------------------------------------


def test_q8_1_invariants(oracle):
    rng = np.random.default_rng(11)
    x = _bf16_round(rng.standard_normal((9, 512)).astype(np.float32) * 3.0)
    x[2, 64:96] = 0.0  # a zero block
    x[3, 0:32] = _bf16_round(np.full(32, 0.0078125, dtype=np.float32))  # constant block
    q, d, s = oracle.quantize_q8_1(_bf16_bits(x))
    blocks = x.reshape(9, 16, 32)
    amax = np.abs(blocks).max(axis=2)
    np.testing.assert_array_equal(d, (amax / np.float32(127.0)).astype(np.float32))
    qb = q.reshape(9, 16, 32).astype(np.int32)
    assert np.abs(qb).max() <= 127
    nonzero = amax > 0
    assert (np.abs(qb).max(axis=2)[nonzero] == 127).all()
    assert (qb[~nonzero] == 0).all() and (d[~nonzero] == 0).all()
    error = np.abs(blocks.astype(np.float64) - d[..., None].astype(np.float64) * qb)
    # d/2 plus the fp32 rounding of x*(127/amax) near a tie
    assert (error <= d[..., None].astype(np.float64) * 0.5 + 1e-6 * amax[..., None]).all()
    np.testing.assert_allclose(s, blocks.astype(np.float64).sum(axis=2), rtol=0, atol=1e-4)
    assert (qb[3, 0] == 127).all()


def test_q8_1_rounds_half_away_from_zero(oracle):
    # amax = 127 makes the scale exactly 1, so x itself is what gets rounded
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :8] = [127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.25]
    q, d, _ = oracle.quantize_q8_1(_bf16_bits(x))
    assert d[0, 0] == 1.0
    assert q[0, :8].tolist() == [127, 1, -1, 2, -2, 3, -3, 0]


def test_q8_1_brute_force(oracle):
    rng = np.random.default_rng(5)
    x = _bf16_round(rng.standard_normal((4, 256)).astype(np.float32))
    q, d, s = oracle.quantize_q8_1(_bf16_bits(x))
    for r in range(4):
        for b in range(8):
            values = x[r, 32 * b : 32 * b + 32]
            amax = np.float32(np.abs(values).max())
            inverse = np.float32(127.0) / amax
            for i in range(32):
                scaled = np.float32(values[i] * inverse)
                rounded = int(np.floor(abs(float(scaled)) + 0.5)) * (1 if scaled >= 0 else -1)
                assert q[r, 32 * b + i] == rounded
            lanes = [np.float32(np.float32(np.float32(values[4 * t] + values[4 * t + 1]) + values[4 * t + 2]) + values[4 * t + 3]) for t in range(8)]
            a = [np.float32(lanes[t] + lanes[t + 4]) for t in range(4)]
            total = np.float32(np.float32(a[0] + a[2]) + np.float32(a[1] + a[3]))
            assert s[r, b] == total


# ---- matmul helpers --------------------------------------------------------------------


def _zeroed_quants(qtype, packed):
    """Copy of Q4_K/Q5_K rows with every quant bit cleared: decodes to -dmin*m."""
    block = {Q4_K: 144, Q5_K: 176}[qtype]
    data = packed.reshape(-1, block).copy()
    data[:, 16:] = 0
    return data.reshape(packed.shape)


@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_mmq_forward_equals_dequantized_operands_matmul(oracle, qtype):
    import synth

    rng = np.random.default_rng(200 + qtype)
    rows, n, k = 5, 7, 512
    packed = synth.random_packed_weight(qtype, (n,), k, seed=qtype).numpy()
    x = _bf16_round(rng.standard_normal((rows, k)).astype(np.float32))
    q, d, s = oracle.quantize_q8_1(_bf16_bits(x))
    x_hat = (q.reshape(rows, k // 32, 32).astype(np.float64) * d[..., None].astype(np.float64)).reshape(rows, k)
    weights = npdecode.dequant_rows(qtype, packed, k, oracle.iq2s_grid()).astype(np.float64)
    expected = x_hat @ weights.T
    if qtype in (Q4_K, Q5_K):
        # w = a*q - b with b = dmin*m per 32 values: the algebra replaces sum(b*x_hat) by b*sum(x)
        minus_b = npdecode.dequant_rows(qtype, _zeroed_quants(qtype, packed), k).astype(np.float64)
        b32 = -minus_b.reshape(n, k // 32, 32)[:, :, 0]
        block_sum_hat = x_hat.reshape(rows, k // 32, 32).sum(axis=2)
        expected = expected + block_sum_hat @ b32.T - s.astype(np.float64) @ b32.T
    actual = oracle.mmq_forward(qtype, _bf16_bits(x), packed, n, k)
    np.testing.assert_allclose(actual, expected, rtol=2e-6, atol=1e-7)


def test_round_to_half_is_numpy_float16(oracle):
    """Every half value, the midpoints between neighbours (ties go to even), values a hair to either side of them,
    the subnormal range, the overflow threshold 65520 and infinities: same result as numpy's float32 -> float16."""
    halves = np.arange(0, 0x7C01, dtype=np.uint16).view(np.float16).astype(np.float32)   # 0 .. inf
    mid = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    probes = np.concatenate([
        halves, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
        np.float32([65519.99, 65520.0, 65520.01, 1e6, 3e38, 5.9e-8, 2.9e-8, 3.0e-8, 1e-10, 0.0]),
    ])
    probes = np.concatenate([probes, -probes])
    with np.errstate(over="ignore"):
        expected = probes.astype(np.float16).astype(np.float32)
    actual = oracle.round_to_half(probes)
    np.testing.assert_array_equal(actual.view(np.uint32), expected.view(np.uint32))


def _k45_fields(qtype, block):
    """(quants[256], sc[8], mn[8], d, dmin) of one Q4_K / Q5_K block, read off the layout with numpy."""
    d = np.frombuffer(bytes(block[0:2]), dtype=np.float16)[0]
    dmin = np.frombuffer(bytes(block[2:4]), dtype=np.float16)[0]
    scales = block[4:16].astype(np.int64)
    sc, mn = np.zeros(8, dtype=np.int64), np.zeros(8, dtype=np.int64)
    for j in range(8):
        if j < 4:
            sc[j], mn[j] = scales[j] & 63, scales[j + 4] & 63
        else:
            sc[j] = (scales[j + 4] & 0x0F) | ((scales[j - 4] >> 6) << 4)
            mn[j] = (scales[j + 4] >> 4) | ((scales[j] >> 6) << 4)
    low = block[16:144] if qtype == Q4_K else block[48:176]
    high = None if qtype == Q4_K else block[16:48]
    quants = np.zeros(256, dtype=np.int64)
    for chunk in range(4):
        nibbles = low[32 * chunk: 32 * chunk + 32].astype(np.int64)
        first, second = nibbles & 0x0F, nibbles >> 4
        if high is not None:
            first = first + 16 * ((high.astype(np.int64) >> (2 * chunk)) & 1)
            second = second + 16 * ((high.astype(np.int64) >> (2 * chunk + 1)) & 1)
        quants[64 * chunk: 64 * chunk + 32] = first
        quants[64 * chunk + 32: 64 * chunk + 64] = second
    return quants, sc, mn, d, dmin


@pytest.mark.parametrize("qtype", (Q4_K, Q5_K))
def test_half_scale_mode_equals_numpy_restatement_and_stays_close_to_fp32_mode(oracle, qtype):
    """The reference keeps four numbers per 32-value block as fp16 for these two formats: d*sc and -dmin*m of the
    weights (a half2 product) and d and sum of the activations.  The oracle's half-scale mode is checked against a numpy
    float64 evaluation with float16 casts in those four places, and its distance from the fp32-scale algebra (what the
    library computes) is measured: a relative error of at most 2^-11 per factor, far inside the 1e-2 the operator
    promises."""
    import synth
    from helpers import max_rel_to_peak, nrmse

    rng = np.random.default_rng(900 + qtype)
    rows, n, k = 6, 9, 1024
    block_bytes = 144 if qtype == Q4_K else 176
    packed = synth.random_packed_weight(qtype, (n,), k, seed=70 + qtype).numpy().reshape(n, k // 256, block_bytes)
    x = _bf16_round(rng.standard_normal((rows, k)).astype(np.float32))
    q, d, s = oracle.quantize_q8_1(_bf16_bits(x))
    d16 = d.astype(np.float16).astype(np.float64)
    s16 = s.astype(np.float16).astype(np.float64)
    expected = np.zeros((rows, n))
    for col in range(n):
        for b in range(k // 256):
            quants, sc, mn, dw, dmin = _k45_fields(qtype, packed[col, b])
            scale = (np.float16(dw) * sc.astype(np.float16)).astype(np.float64)       # half multiply
            minimum = (np.float16(-dmin) * mn.astype(np.float16)).astype(np.float64)
            for g in range(8):
                block = 8 * b + g
                dot = q[:, 32 * block: 32 * block + 32].astype(np.int64) @ quants[32 * g: 32 * g + 32]
                expected[:, col] += scale[g] * d16[:, block] * dot + minimum[g] * s16[:, block]
    half_mode = oracle.mmq_forward_half_scales(qtype, _bf16_bits(x), packed, n, k)
    np.testing.assert_allclose(half_mode, expected, rtol=2e-6, atol=1e-6)
    fp32_mode = oracle.mmq_forward(qtype, _bf16_bits(x), packed, n, k)
    assert nrmse(fp32_mode, half_mode) < 1e-3
    assert max_rel_to_peak(fp32_mode, half_mode) < 1e-3


@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_linear_and_grad_input_equal_float64_matmul(oracle, qtype):
    import synth

    rng = np.random.default_rng(300 + qtype)
    rows, n, k = 4, 9, 256
    packed = synth.random_packed_weight(qtype, (n,), k, seed=50 + qtype).numpy()
    weights = _bf16_round(npdecode.dequant_rows(qtype, packed, k, oracle.iq2s_grid())).astype(np.float64)
    x = _bf16_round(rng.standard_normal((rows, k)).astype(np.float32))
    dy = _bf16_round(rng.standard_normal((rows, n)).astype(np.float32))
    np.testing.assert_allclose(
        oracle.linear_forward(qtype, _bf16_bits(x), packed, n, k), x.astype(np.float64) @ weights.T, rtol=1e-6, atol=1e-9
    )
    np.testing.assert_allclose(
        oracle.grad_input(qtype, _bf16_bits(dy), packed, n, k), dy.astype(np.float64) @ weights, rtol=1e-6, atol=1e-9
    )


@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_one_hot_cotangent_reproduces_weight_row(oracle, qtype):
    import synth

    packed = synth.random_packed_weight(qtype, (5,), 512, seed=80 + qtype).numpy()
    dy = np.zeros((1, 5), dtype=np.float32)
    dy[0, 3] = 1.0
    result = oracle.grad_input(qtype, _bf16_bits(dy), packed, 5, 512)
    # compared as values: an accumulator that starts at +0 turns a decoded -0 into +0
    np.testing.assert_array_equal(
        oracle.bf16_to_f32(oracle.f32_to_bf16(result)[0]),
        oracle.bf16_to_f32(oracle.dequant_bf16(qtype, packed, 512)[3]),
    )


def test_grouped_helper_skips_invalid_groups(oracle):
    import synth

    packed = synth.random_packed_weight(Q4_K, (3, 4), 256, seed=1).numpy()
    x = _bf16_bits(np.ones((6, 256), dtype=np.float32))
    out = oracle.grouped(oracle.linear_forward, Q4_K, x, packed, [0, 7, 2], [2, 4, 6], 4, 256, 4)
    assert np.isfinite(out[0:2]).all() and np.isnan(out[2:4]).all() and np.isfinite(out[4:6]).all()
    np.testing.assert_array_equal(out[4:6], oracle.linear_forward(Q4_K, x[4:6], packed[2], 4, 256))


def test_round_half_up_equals_roundf_on_every_product_the_quantizer_can_form():
    """The GPU quantizer rounds |x * (127 / amax)| with the hardware's round-half-up conversion, the reference with
    roundf (csrc/mmq_core.cuh:186).  On non-negative inputs the two differ at one float only, the largest one below
    0.5 (0x3EFFFFFF), if the conversion adds 0.5 in fp32.  x and amax are bf16 values and powers of two cancel in the
    product, so all products are covered by amax in [1, 2) and x <= amax: none of them is that float."""
    target = np.array([0x3EFFFFFF], dtype=np.uint32).view(np.float32)[0]
    mantissas = (1.0 + np.arange(128, dtype=np.float64) / 128.0)
    amax = mantissas.astype(np.float32)                                   # [128]
    d_inv = (np.float32(127.0) / amax).astype(np.float32)
    exponents = 2.0 ** np.arange(-140, 1, dtype=np.float64)
    x = (mantissas[None, :] * exponents[:, None]).astype(np.float32).reshape(-1)   # every bf16 magnitude below 2
    product = (x[None, :] * d_inv[:, None]).astype(np.float32)
    reachable = x[None, :] <= amax[:, None]
    assert not np.any(reachable & (product == target))
