"""GPU tests of the mixture-of-experts steps around the grouped operators (-m gpu): routing sort,
routing-weighted combine, and the whole SwiGLU layer against a float64 restatement on dequantized weights.

The reference leaves these steps to its callers, so the expected values here are plain
index arithmetic in float64 (combine) and the oracle's scalar dequantizer followed by dense
float64 matmuls (layer).
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


def _choices(tokens, top_k, experts, seed):
    generator = np.random.default_rng(seed)
    chosen = np.stack([generator.permutation(experts)[:top_k] for _ in range(tokens)])
    weights = generator.random((tokens, top_k), dtype=np.float32) + 0.1
    weights /= weights.sum(axis=1, keepdims=True)
    return torch.from_numpy(chosen).cuda(), torch.from_numpy(weights).cuda()


def test_route_sorts_slots_by_expert(ops):
    tgo, _ = ops
    slot_experts, _ = _choices(33, 4, 9, seed=1)
    row_index, slot_rows, indices, offsets = tgo.route(slot_experts, 9)
    flat = slot_experts.reshape(-1).cpu().numpy()
    order = np.argsort(flat, kind="stable")
    assert np.array_equal(row_index.cpu().numpy(), order // 4)
    assert np.array_equal(slot_rows.reshape(-1).cpu().numpy()[order], np.arange(flat.size))
    assert np.array_equal(offsets.cpu().numpy(), np.cumsum(np.bincount(flat, minlength=9)))
    assert indices.tolist() == list(range(9)) and offsets.dtype == torch.int32


@pytest.mark.parametrize("tokens,top_k,experts", ((1, 1, 1), (1, 8, 256), (8, 8, 256), (512, 8, 256), (3, 5, 4096),
                                                    (300, 7, 3), (513, 8, 256), (1000, 8, 64)))
def test_route_of_any_size_is_the_stable_sort(ops, tokens, top_k, experts):
    """Up to 4096 slots are sorted by one kernel launch (tgo_route_small), more by tensor operations: either way the
    result is the stable sort by expert (numpy's), with one group per expert."""
    tgo, _ = ops
    generator = np.random.default_rng(tokens * 31 + experts)
    flat = generator.integers(0, experts, size=tokens * top_k)
    if tokens * top_k > 20:
        flat[5:15] = flat[5]          # a run of one expert
    slot_experts = torch.from_numpy(flat.reshape(tokens, top_k)).cuda()
    row_index, slot_rows, indices, offsets = tgo.route(slot_experts, experts)
    order = np.argsort(flat, kind="stable")
    assert row_index.dtype == torch.int64 and slot_rows.dtype == torch.int64 and slot_rows.shape == (tokens, top_k)
    assert np.array_equal(row_index.cpu().numpy(), order // top_k)
    assert np.array_equal(slot_rows.reshape(-1).cpu().numpy()[order], np.arange(flat.size))
    assert np.array_equal(offsets.cpu().numpy(), np.cumsum(np.bincount(flat, minlength=experts)))
    assert indices.tolist() == list(range(experts)) and offsets.dtype == torch.int32 and indices.dtype == torch.int64


@pytest.mark.parametrize("tokens,top_k,features", ((1, 1, 8), (7, 3, 200), (64, 8, 2048), (5, 6, 4104)))
def test_combine_matches_float64(ops, tokens, top_k, features):
    tgo, _ = ops
    num_rows = tokens * top_k
    rows = random_bf16((num_rows, features), seed=features)
    generator = np.random.default_rng(tokens)
    slot_rows = torch.from_numpy(generator.permutation(num_rows).reshape(tokens, top_k)).cuda()
    weights = torch.from_numpy(generator.standard_normal((tokens, top_k)).astype(np.float32)).cuda()
    out = tgo.moe_combine(rows, slot_rows, weights)
    assert out.shape == (tokens, features) and out.dtype == torch.bfloat16
    expected = (rows.double()[slot_rows] * weights.double().unsqueeze(-1)).sum(dim=1)
    assert_matches_f32_reference(out, expected.float().cpu().numpy(), accumulate_noise=1e-6)
    # deterministic: a second call gives the same bits
    torch.testing.assert_close(tgo.moe_combine(rows, slot_rows, weights), out, rtol=0, atol=0)


def test_combine_skips_slots_without_a_row(ops):
    tgo, _ = ops
    rows = random_bf16((6, 64), seed=3)
    slot_rows = torch.tensor([[0, -1], [7, 2], [5, 5]], device="cuda", dtype=torch.int64)
    weights = torch.tensor([[0.5, 9.0], [9.0, 2.0], [1.0, 0.25]], device="cuda")
    out = tgo.moe_combine(rows, slot_rows, weights)
    r = rows.double()
    expected = torch.stack([0.5 * r[0], 2.0 * r[2], 1.25 * r[5]])
    assert_matches_f32_reference(out, expected.float().cpu().numpy(), accumulate_noise=1e-6)


def test_combine_gradients(ops):
    tgo, _ = ops
    tokens, top_k, features = 9, 3, 128
    num_rows = tokens * top_k
    generator = np.random.default_rng(5)
    slot_rows = torch.from_numpy(generator.permutation(num_rows).reshape(tokens, top_k)).cuda()
    rows = random_bf16((num_rows, features), seed=6).requires_grad_(True)
    weights = torch.from_numpy(generator.standard_normal((tokens, top_k)).astype(np.float32)).cuda().requires_grad_(True)
    grad = random_bf16((tokens, features), seed=7)
    tgo.moe_combine(rows, slot_rows, weights).backward(grad)

    rows64 = rows.detach().double().requires_grad_(True)
    weights64 = weights.detach().double().requires_grad_(True)
    (rows64[slot_rows] * weights64.unsqueeze(-1)).sum(dim=1).backward(grad.double())
    assert_matches_f32_reference(rows.grad, rows64.grad.float().cpu().numpy(), accumulate_noise=1e-6)
    torch.testing.assert_close(weights.grad.double(), weights64.grad, rtol=1e-5, atol=1e-5)


def test_combine_rejects_bad_arguments(ops):
    tgo, _ = ops
    rows = random_bf16((4, 64), seed=1)
    slots = torch.zeros((2, 2), device="cuda", dtype=torch.int64)
    weights = torch.ones((2, 2), device="cuda")
    with pytest.raises(RuntimeError, match="slot_weights must have dtype torch.float32"):
        tgo.moe_combine(rows, slots, weights.bfloat16())
    with pytest.raises(RuntimeError, match="shape \\[tokens, top_k\\]"):
        tgo.moe_combine(rows, slots, weights[:1].contiguous())
    with pytest.raises(RuntimeError, match="multiple of 8"):
        tgo.moe_combine(random_bf16((4, 12), seed=2), slots, weights)


@pytest.mark.parametrize("gate_up,down", (("Q4_K", "Q6_K"), ("IQ2_S", "Q5_K")))
def test_layer_matches_float64_on_dequantized_weights(ops, oracle, gate_up, down):
    tgo, synth = ops
    tokens, top_k, experts, features, intermediate = 48, 2, 6, 512, 256
    gate_host = synth.random_packed_weight(QTYPES[gate_up], (experts, intermediate), features, seed=61)
    up_host = synth.random_packed_weight(QTYPES[gate_up], (experts, intermediate), features, seed=62)
    down_host = synth.random_packed_weight(QTYPES[down], (experts, features), intermediate, seed=63)
    hidden = random_bf16((tokens, features), seed=64).requires_grad_(True)
    slot_experts, slot_weights = _choices(tokens, top_k, experts, seed=65)
    out = tgo.moe_layer(
        hidden, slot_experts, slot_weights, gate_host.cuda(), up_host.cuda(), down_host.cuda(),
        QTYPES[gate_up], QTYPES[down], intermediate,
    )
    assert out.shape == (tokens, features)

    def dense(host, qtype, width):
        return torch.from_numpy(
            np.stack([oracle.dequant_f32(qtype, host[e].numpy(), width) for e in range(experts)])
        ).double()

    gate64, up64, down64 = dense(gate_host, QTYPES[gate_up], features), dense(up_host, QTYPES[gate_up], features), dense(down_host, QTYPES[down], intermediate)
    x = hidden.detach().double().cpu().requires_grad_(True)
    expected = torch.zeros((tokens, features), dtype=torch.float64)
    chosen, weight = slot_experts.cpu(), slot_weights.double().cpu()
    for t in range(tokens):
        for j in range(top_k):
            e = int(chosen[t, j])
            inner = torch.nn.functional.silu(gate64[e] @ x[t]) * (up64[e] @ x[t])
            expected[t] = expected[t] + weight[t, j] * (down64[e] @ inner)
    # q8_1 activations and three bf16 roundings along the way: the operators' own tolerance, twice over
    assert nrmse(f32(out), expected.detach().float().numpy()) < 2e-2

    grad = random_bf16((tokens, features), seed=66)
    out.backward(grad)
    expected.backward(grad.double().cpu())
    assert nrmse(f32(hidden.grad), x.grad.float().numpy()) < 2e-2


@pytest.mark.parametrize("qname", ("Q4_K", "Q6_K"))
def test_projection_with_combine_equals_the_two_steps(ops, oracle, qname):
    """grouped_mmq_combine = moe_combine(grouped_mmq(...)): same bits forward, and a backward whose cotangent
    packing gathers the per-token gradient and applies the routing weight itself.  Checked against the two
    separate operators bit for bit, and against a float64 restatement on oracle-dequantized weights."""
    tgo, synth = ops
    qtype, tokens, top_k, experts, k, n = QTYPES[qname], 150, 3, 7, 512, 200
    host = synth.random_packed_weight(qtype, (experts, n), k, seed=71)
    weight = host.cuda()
    slot_experts, slot_weights = _choices(tokens, top_k, experts, seed=72)
    _row_index, slot_rows, indices, offsets = tgo.route(slot_experts, experts)
    rows = tokens * top_k
    grad = random_bf16((tokens, n), seed=74)

    fused_in = random_bf16((rows, k), seed=73).requires_grad_(True)
    fused_w = slot_weights.clone().requires_grad_(True)
    fused = tgo.grouped_mmq_combine(fused_in, weight, indices, offsets, slot_rows, fused_w, qtype, n)
    fused.backward(grad)

    plain_in = random_bf16((rows, k), seed=73).requires_grad_(True)
    plain_w = slot_weights.clone().requires_grad_(True)
    plain = tgo.moe_combine(tgo.grouped_mmq(plain_in, weight, indices, offsets, qtype, n), slot_rows, plain_w)
    plain.backward(grad)

    torch.testing.assert_close(fused, plain, rtol=0, atol=0)
    torch.testing.assert_close(fused_in.grad, plain_in.grad, rtol=0, atol=0)
    torch.testing.assert_close(fused_w.grad, plain_w.grad, rtol=0, atol=0)

    # d/d(input row r) = w[r] * grad[token of r] @ bf16(W[expert of r]), the cotangent rounded to bf16 first
    dense = np.stack([oracle.bf16_to_f32(oracle.dequant_bf16(qtype, host[e].numpy(), k)) for e in range(experts)]).astype(np.float64)
    slot_of_row = np.empty(rows, dtype=np.int64)
    slot_of_row[slot_rows.reshape(-1).cpu().numpy()] = np.arange(rows)
    grad64, weights64 = grad.double().cpu().numpy(), slot_weights.double().cpu().numpy().reshape(-1)
    expert_of_slot = slot_experts.reshape(-1).cpu().numpy()
    expected = np.empty((rows, k))
    for r in range(rows):
        slot = slot_of_row[r]
        cotangent = (torch.from_numpy(weights64[slot] * grad64[slot // top_k]).float().bfloat16().double().numpy())
        expected[r] = cotangent @ dense[expert_of_slot[slot]]
    assert_matches_f32_reference(fused_in.grad, expected.astype(np.float32), accumulate_noise=2e-6)


def test_weighted_grad_input_skips_rows_without_a_token(ops):
    tgo, synth = ops
    qtype, k, n = 12, 256, 64
    weight = synth.random_packed_weight(qtype, (2, n), k, seed=75).cuda()
    grad_tokens = random_bf16((3, n), seed=76)
    row_token = torch.tensor([2, -1, 0, 5, 1], device="cuda", dtype=torch.int64)
    row_weight = torch.tensor([0.5, 3.0, 2.0, 7.0, 1.0], device="cuda")
    indices = torch.tensor([1, 0], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([2, 5], device="cuda", dtype=torch.int32)
    actual = torch.ops.torch_ggml_ops.grouped_mmq_grad_input_weighted.default(
        grad_tokens, row_token, row_weight, weight, indices, offsets, qtype, k
    )
    sorted_grad = torch.zeros((5, n), device="cuda", dtype=torch.bfloat16)
    for row, (token, factor) in enumerate(zip(row_token.tolist(), row_weight.tolist())):
        if 0 <= token < 3:
            sorted_grad[row] = (grad_tokens[token].float() * factor).bfloat16()
    expected = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(sorted_grad, weight, indices, offsets, qtype, k)
    torch.testing.assert_close(actual, expected, rtol=0, atol=0)
    assert torch.count_nonzero(actual[1]) == 0 and torch.count_nonzero(actual[3]) == 0
    with pytest.raises(RuntimeError, match="row_weight"):
        torch.ops.torch_ggml_ops.grouped_mmq_grad_input_weighted.default(
            grad_tokens, row_token, row_weight.double(), weight, indices, offsets, qtype, k
        )
