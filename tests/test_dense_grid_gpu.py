"""Every cell of the dense parity grid at its exact shape (-m gpu).

Five formats x M in {1, 16, 512, 4096} x N in {2048, 4096}, K = 2048, forward and grad-input, plus the
Q4_K M = 32, N = K = 2048 case.  Each (M, N) selects its own kernel family or tile shape in the launchers
(GEMV up to 32 rows, 32-row narrow tiles or reduced tiles when full tiles cannot fill the chip, split
reductions for the grad-input of few rows), so each one is run, mirroring the reference's
tests/test_mmq.py:50-118 with seeded synthetic blocks:

* homogeneity at the full shape: doubling the activations (or the cotangent) doubles every bf16 result bit
  for bit, because q8_1 block scales and sums (resp. the bf16 cotangent) double exactly;
* the oracle on a sample of rows that includes the edges of the 32-, 128- and 256-row tiles and the last row:
  same algebra in float64 up to fp32 accumulation and the final rounding, and within the stated 1e-2 of the
  dequantize-then-matmul path (NRMSE and max error over max reference).
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits, f32, forward_noise, max_rel_to_peak, nrmse

pytestmark = pytest.mark.gpu

K = 2048
FORWARD_TOLERANCE = 1e-2   # against x @ bf16(W)^T, on norms
EDGE_ROWS = (0, 1, 31, 32, 33, 63, 64, 127, 128, 129, 255, 256, 257, 511, 512, 2047, 2048, 4064)


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


_weights = {}


def _weight(synth, qtype, n):
    """One seeded weight per (format, N), shared by the cells of that column."""
    key = (qtype, n)
    if key not in _weights:
        host = synth.random_packed_weight(qtype, (n,), K, seed=9000 + 10 * qtype + n // 2048)
        _weights[key] = (host.numpy(), host.cuda())
    return _weights[key]


def _sample(m, seed):
    rows = {r for r in EDGE_ROWS if r < m} | {m - 1}
    rng = np.random.default_rng(seed)
    while len(rows) < min(m, 20):
        rows.add(int(rng.integers(0, m)))
    return sorted(rows)


def _check_forward(tgo, oracle, qtype, x, packed_host, packed, n, rows):
    out = tgo.mmq(x, packed, qtype, n)
    assert out.shape == (x.shape[0], n) and out.dtype == torch.bfloat16 and out.is_contiguous()
    torch.testing.assert_close(tgo.mmq(x * 2, packed, qtype, n), out * 2, rtol=0, atol=0)
    index = torch.tensor(rows, device="cuda")
    x_rows = bits(x.index_select(0, index))
    picked = out.index_select(0, index)
    assert_matches_f32_reference(picked, oracle.mmq_forward(qtype, x_rows, packed_host, n, K), forward_noise(qtype, x.shape[0], n))
    expected = oracle.linear_forward(qtype, x_rows, packed_host, n, K)
    assert nrmse(f32(picked), expected) < FORWARD_TOLERANCE
    assert max_rel_to_peak(f32(picked), expected) < FORWARD_TOLERANCE


def _check_grad_input(oracle, qtype, dy, packed_host, packed, n, rows):
    op = torch.ops.torch_ggml_ops.mmq_grad_input.default
    grad = op(dy, packed, qtype, K)
    assert grad.shape == (dy.shape[0], K) and grad.dtype == torch.bfloat16 and grad.is_contiguous()
    torch.testing.assert_close(op(dy * 2, packed, qtype, K), grad * 2, rtol=0, atol=0)
    index = torch.tensor(rows, device="cuda")
    expected = oracle.grad_input(qtype, bits(dy.index_select(0, index)), packed_host, n, K)
    # fp32 accumulation of exact bf16 products: only the final rounding separates it from float64
    assert_matches_f32_reference(grad.index_select(0, index), expected, accumulate_noise=2e-6)


@pytest.mark.parametrize("n", (2048, 4096))
@pytest.mark.parametrize("m", (1, 16, 512, 4096))
@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_dense_grid_cell(ops, oracle, qname, m, n):
    tgo, synth = ops
    qtype = QTYPES[qname]
    packed_host, packed = _weight(synth, qtype, n)
    generator = torch.Generator(device="cuda").manual_seed(1000 * m + n + qtype)
    x = torch.randn(m, K, device="cuda", generator=generator).to(torch.bfloat16)
    dy = torch.randn(m, n, device="cuda", generator=generator).to(torch.bfloat16)
    rows = _sample(m, seed=m + n)
    _check_forward(tgo, oracle, qtype, x, packed_host, packed, n, rows)
    _check_grad_input(oracle, qtype, dy, packed_host, packed, n, rows)


def test_q4k_32_rows_square_against_the_oracle_everywhere(ops, oracle):
    """Q4_K, M = 32, N = K = 2048 (the configuration the CPU path is timed on): every row, both directions."""
    tgo, synth = ops
    qtype, m, n = QTYPES["Q4_K"], 32, 2048
    host = synth.random_packed_weight(qtype, (n,), K, seed=4242)
    packed_host, packed = host.numpy(), host.cuda()
    generator = torch.Generator(device="cuda").manual_seed(32)
    x = torch.randn(m, K, device="cuda", generator=generator).to(torch.bfloat16)
    dy = torch.randn(m, n, device="cuda", generator=generator).to(torch.bfloat16)
    _check_forward(tgo, oracle, qtype, x, packed_host, packed, n, list(range(m)))
    _check_grad_input(oracle, qtype, dy, packed_host, packed, n, list(range(m)))
