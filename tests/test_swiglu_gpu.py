"""GPU parity of the gate/up pair with the fused SwiGLU epilogue (-m gpu).

The reference's pair operator ends at the two projections, so the expected values are built from the
library's own ``grouped_mmq_pair`` (pinned against the CPU oracle elsewhere): the fused operator's gate
must equal the pair's gate bit for bit, and its result must equal ``silu(gate) * up`` evaluated in float64
from the pair's bf16 outputs, up to the single final rounding.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, f32, nrmse, random_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


def _metadata(experts, offsets):
    return (
        torch.tensor(experts, device="cuda", dtype=torch.int64),
        torch.tensor(offsets, device="cuda", dtype=torch.int32),
    )


def _expected(gate, up):
    g, u = gate.double(), up.double()
    return (g / (1.0 + torch.exp(-g)) * u).float().cpu().numpy()


# group sizes cover narrow tasks (<= 32 rows), partial and full row tiles and a group spanning several tiles
SIZES = [300, 7, 33, 1, 128, 64, 31, 32]
EXPERTS = [5, 0, 3, 7, 1, 6, 2, 4]


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_fused_activation_against_the_oracle(ops, oracle, qname):
    """Independent of the library's own pair operator: gate and up from the CPU oracle's forward algebra (float64
    accumulation), the gate rounded to bf16 as the operator stores it, silu(gate) * up in float64.  The fused result
    may differ from that by the rounding of its own gate (one bf16 ulp of the gate, passed through silu') and its own
    final rounding, so the comparison is on norms, like the forward's stated tolerance."""
    from helpers import bits, max_rel_to_peak

    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 96, 512
    offsets = np.cumsum(SIZES).tolist()
    rows = offsets[-1]
    gate_host = synth.random_packed_weight(qtype, (8, n), k, seed=300 + qtype)
    up_host = synth.random_packed_weight(qtype, (8, n), k, seed=310 + qtype)
    x = random_bf16((rows, k), seed=77)
    metadata = _metadata(EXPERTS, offsets)
    activated = tgo.grouped_mmq_swiglu(x, gate_host.cuda(), up_host.cuda(), *metadata, qtype, n)
    gate = oracle.grouped(oracle.mmq_forward, qtype, bits(x), gate_host.numpy(), EXPERTS, offsets, n, k, n)
    up = oracle.grouped(oracle.mmq_forward, qtype, bits(x), up_host.numpy(), EXPERTS, offsets, n, k, n)
    gate_bf16 = torch.from_numpy(gate).to(torch.bfloat16).double().numpy()
    with np.errstate(over="ignore"):   # exp(-gate) of a large negative gate: the quotient is then exactly 0
        expected = gate_bf16 / (1.0 + np.exp(-gate_bf16)) * up.astype(np.float64)
    assert nrmse(f32(activated), expected) < 5e-3
    assert max_rel_to_peak(f32(activated), expected) < 1e-2


@pytest.fixture(params=("auto", "scaled"))
def operand(request):
    """"scaled": the kind that large calls take by themselves, whose kernel stores both projections and leaves the
    activation to an elementwise pass; forced here so that the small shapes below reach it."""
    from torch_ggml_ops import _native

    _native.set_forward_operand(request.param)
    yield request.param
    _native.set_forward_operand("auto")


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize("n", (512, 96, 37))
def test_fused_activation_matches_pair_then_swiglu(ops, operand, qname, n):
    """n = 512: whole tiles; 96: a partial column tile; 37: odd row stride, element-wise stores."""
    tgo, synth = ops
    qtype, k = QTYPES[qname], 512
    offsets = np.cumsum(SIZES).tolist()
    rows = offsets[-1]
    gate_w = synth.random_packed_weight(qtype, (8, n), k, seed=300 + qtype).cuda()
    up_w = synth.random_packed_weight(qtype, (8, n), k, seed=310 + qtype).cuda()
    x = random_bf16((rows, k), seed=n)
    metadata = _metadata(EXPERTS, offsets)
    activated, gate, _kept_up = torch.ops.torch_ggml_ops.grouped_mmq_swiglu.default(x, None, gate_w, up_w, *metadata, qtype, n)
    plain_gate, plain_up = tgo.grouped_mmq_pair(x, gate_w, up_w, *metadata, qtype, n)
    torch.testing.assert_close(gate, plain_gate, rtol=0, atol=0)
    assert_matches_f32_reference(activated, _expected(plain_gate, plain_up), accumulate_noise=1e-6)
    torch.testing.assert_close(tgo.grouped_mmq_swiglu(x, gate_w, up_w, *metadata, qtype, n), activated, rtol=0, atol=0)


def test_fused_activation_from_token_rows(ops, operand):
    tgo, synth = ops
    qtype, n, k, tokens, top_k, experts = 13, 256, 1024, 120, 4, 8
    gate_w = synth.random_packed_weight(qtype, (experts, n), k, seed=41).cuda()
    up_w = synth.random_packed_weight(qtype, (experts, n), k, seed=42).cuda()
    hidden = random_bf16((tokens, k), seed=43)
    generator = np.random.default_rng(44)
    chosen = torch.from_numpy(np.stack([generator.permutation(experts)[:top_k] for _ in range(tokens)])).cuda()
    row_index, _, indices, offsets = tgo.route(chosen, experts)
    activated = tgo.grouped_mmq_swiglu(hidden, gate_w, up_w, indices, offsets, qtype, n, row_index)
    gate, up = tgo.grouped_mmq_pair(hidden.index_select(0, row_index), gate_w, up_w, indices, offsets, qtype, n)
    assert activated.shape == (tokens * top_k, n)
    assert_matches_f32_reference(activated, _expected(gate, up), accumulate_noise=1e-6)


def test_extreme_gates_saturate_cleanly(ops):
    """Large |gate|: silu(g) -> g for g >> 0 and -> 0 for g << 0 (exp overflow must not produce NaN)."""
    tgo, synth = ops
    qtype, n, k = 12, 64, 256
    gate_w = synth.random_packed_weight(qtype, (1, n), k, seed=51).cuda()
    up_w = synth.random_packed_weight(qtype, (1, n), k, seed=52).cuda()
    x = random_bf16((40, k), seed=53, scale=3000.0)
    metadata = _metadata([0], [40])
    activated, gate, _kept_up = torch.ops.torch_ggml_ops.grouped_mmq_swiglu.default(x, None, gate_w, up_w, *metadata, qtype, n)
    _, up = tgo.grouped_mmq_pair(x, gate_w, up_w, *metadata, qtype, n)
    assert torch.isfinite(activated).all() and gate.float().abs().max() > 100.0
    assert_matches_f32_reference(activated, _expected(gate, up), accumulate_noise=1e-6)


@pytest.mark.parametrize("gathered", (False, True))
def test_gradient_matches_the_unfused_chain(ops, operand, gathered):
    """(with the scaled operands the operator keeps the up projection for the backward pass, otherwise it computes it
    again there: both routes are compared with the unfused chain)"""
    tgo, synth = ops
    qtype, n, k, experts = 13, 128, 512, 6
    gate_w = synth.random_packed_weight(qtype, (experts, n), k, seed=61).cuda()
    up_w = synth.random_packed_weight(qtype, (experts, n), k, seed=62).cuda()
    tokens, top_k = 60, 3
    generator = np.random.default_rng(63)
    chosen = torch.from_numpy(np.stack([generator.permutation(experts)[:top_k] for _ in range(tokens)])).cuda()
    row_index, _, indices, offsets = tgo.route(chosen, experts)
    hidden = random_bf16((tokens, k), seed=64)
    source = hidden if gathered else hidden.index_select(0, row_index)
    grad = random_bf16((tokens * top_k, n), seed=65)

    fused_in = source.clone().requires_grad_(True)
    activated, _, kept_up = torch.ops.torch_ggml_ops.grouped_mmq_swiglu.default(
        fused_in, row_index if gathered else None, gate_w, up_w, indices, offsets, qtype, n
    )
    assert kept_up.shape == ((tokens * top_k, n) if operand == "scaled" else (0, n))
    activated.backward(grad)

    plain_in = source.clone().requires_grad_(True)
    if gathered:
        gate, up = tgo.grouped_mmq_pair_gathered(plain_in, row_index, gate_w, up_w, indices, offsets, qtype, n)
    else:
        gate, up = tgo.grouped_mmq_pair(plain_in, gate_w, up_w, indices, offsets, qtype, n)
    (torch.nn.functional.silu(gate.float()) * up.float()).backward(grad.float())
    assert fused_in.grad.shape == plain_in.grad.shape
    # both chains round d_gate and d_up to bf16 before the grad-input kernel, at slightly different points
    assert nrmse(f32(fused_in.grad), f32(plain_in.grad)) < 1e-2


@pytest.mark.parametrize("count", (8 * 1000, 4099))
@pytest.mark.parametrize("direct", (False, True))
def test_activation_backward_kernel_matches_the_formulas(ops, count, direct):
    """tgo_swiglu_backward against the same formulas written with fp32 tensor operations: d_up = dy * gate * s and
    d_gate = dy * up * s * (1 + gate * (1 - s)) (+ a cotangent of the gate itself), rounded to bf16 once.  The kernel's
    sigmoid uses the hardware's exponential and reciprocal, so a result may land on the neighbouring bf16 value: the
    bound is one bf16 step (2^-7 relative), and large gates of either sign must stay finite."""
    from torch_ggml_ops import swiglu as module

    generator = torch.Generator(device="cuda").manual_seed(count)
    gate = (4.0 * torch.randn(count, device="cuda", generator=generator)).to(torch.bfloat16)
    gate[:6] = torch.tensor([0.0, -0.0, 60.0, -60.0, 200.0, -200.0], dtype=torch.bfloat16)
    up = torch.randn(count, device="cuda", generator=generator).to(torch.bfloat16)
    dy = torch.randn(count, device="cuda", generator=generator).to(torch.bfloat16)
    grad_gate = torch.randn(count, device="cuda", generator=generator).to(torch.bfloat16) if direct else None
    if count % 8:   # an odd length and a start off the 16-byte grid: the element-at-a-time path
        gate, up, dy = gate[1:], up[1:], dy[1:]
        grad_gate = None if grad_gate is None else grad_gate[1:]
    d_gate, d_up = module._activation_backward(gate, up, dy, grad_gate)
    g, u, y = gate.float(), up.float(), dy.float()
    s = torch.sigmoid(g)
    expected_up = y * (g * s)
    expected_gate = y * u * (s * (1.0 + g * (1.0 - s))) + (0.0 if grad_gate is None else grad_gate.float())
    assert torch.isfinite(d_gate).all() and torch.isfinite(d_up).all()
    for actual, expected in ((d_up, expected_up), (d_gate, expected_gate)):
        error = (actual.float() - expected).abs()
        assert bool((error <= 2.0**-7 * expected.abs() + 1e-30).all()), float((error / expected.abs().clamp_min(1e-30)).max())
