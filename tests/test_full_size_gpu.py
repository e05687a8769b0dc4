"""The benchmark configurations at their full sizes (-m gpu).

The oracle cannot evaluate 65 536 rows against 256 experts in test time, so these sizes are covered by
(a) properties that hold exactly whatever the size, and (b) the oracle on a sample of rows that includes the
first and last row of small, partial and multi-tile groups:

* homogeneity: scaling the activations (or the cotangent) by 2 scales every q8_1 block scale and sum (resp.
  every bf16 cotangent) by exactly 2 and leaves the integer parts alone, so the bf16 results double bit for bit;
* the fused pair equals two single calls, and the pair grad-input equals what the single grad-inputs sum to
  in exact arithmetic (checked on the sample in float64);
* rows are independent: reversing the rows inside every expert group reverses the outputs inside the group.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits, forward_noise

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


def _sample_rows(offsets, rng, per_kind=6):
    """Rows worth checking: the edges and a middle row of the smallest, a few random and the largest groups."""
    ends = np.asarray(offsets, dtype=np.int64)
    starts = np.concatenate([[0], ends[:-1]])
    sizes = ends - starts
    order = np.argsort(sizes)
    groups = set(order[:per_kind].tolist()) | set(order[-per_kind:].tolist())
    groups |= set(rng.choice(len(sizes), size=min(per_kind, len(sizes)), replace=False).tolist())
    rows = []
    for g in sorted(groups):
        if sizes[g] > 0:
            rows += [(g, int(starts[g])), (g, int(ends[g] - 1)), (g, int(starts[g] + sizes[g] // 2))]
    return sorted(set(rows), key=lambda item: item[1])


def _reverse_within_groups(offsets, rows):
    ends = np.asarray(offsets, dtype=np.int64)
    starts = np.concatenate([[0], ends[:-1]])
    index = np.arange(rows)
    for begin, end in zip(starts, ends):
        index[begin:end] = index[begin:end][::-1]
    return torch.from_numpy(index).cuda()


@pytest.mark.parametrize("qname", ("Q5_K", "IQ2_S"))
def test_pair_forward_and_backward_at_the_benchmark_size(ops, oracle, qname):
    """256 experts, gate and up [512, 2048] (Q5_K: the benchmark's format; IQ2_S: the format the reference's model packs
    them in), 8192 tokens x top-8 with Zipf-skewed routing (65 536 rows)."""
    tgo, synth = ops
    qtype, n, k, experts = QTYPES[qname], 512, 2048, 256
    token_of_row, indices, offsets, _ = synth.zipf_routing(8192, experts, 8, 2024, device="cuda")
    rows = token_of_row.numel()
    assert rows == 65536
    generator = torch.Generator(device="cuda").manual_seed(7)
    hidden = torch.randn(8192, k, device="cuda", generator=generator).to(torch.bfloat16)
    x = hidden.index_select(0, token_of_row).contiguous()
    gate = synth.random_packed_weight(qtype, (experts, n), k, 71, device="cuda")
    up = synth.random_packed_weight(qtype, (experts, n), k, 72, device="cuda")
    out_gate, out_up = tgo.grouped_mmq_pair(x, gate, up, indices, offsets, qtype, n)

    torch.testing.assert_close(tgo.grouped_mmq(x, gate, indices, offsets, qtype, n), out_gate, rtol=0, atol=0)
    torch.testing.assert_close(tgo.grouped_mmq(x, up, indices, offsets, qtype, n), out_up, rtol=0, atol=0)
    doubled_gate, doubled_up = tgo.grouped_mmq_pair(x * 2, gate, up, indices, offsets, qtype, n)
    torch.testing.assert_close(doubled_gate, out_gate * 2, rtol=0, atol=0)
    torch.testing.assert_close(doubled_up, out_up * 2, rtol=0, atol=0)
    flip = _reverse_within_groups(offsets.cpu().numpy(), rows)
    flipped_gate, _ = tgo.grouped_mmq_pair(x.index_select(0, flip), gate, up, indices, offsets, qtype, n)
    torch.testing.assert_close(flipped_gate, out_gate.index_select(0, flip), rtol=0, atol=0)
    gathered_gate, gathered_up = tgo.grouped_mmq_pair_gathered(hidden, token_of_row, gate, up, indices, offsets, qtype, n)
    torch.testing.assert_close(gathered_gate, out_gate, rtol=0, atol=0)
    torch.testing.assert_close(gathered_up, out_up, rtol=0, atol=0)

    grad_gate = torch.randn(rows, n, device="cuda", generator=generator).to(torch.bfloat16)
    grad_up = torch.randn(rows, n, device="cuda", generator=generator).to(torch.bfloat16)
    pair_grad = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
        grad_gate, grad_up, gate, up, indices, offsets, qtype, k
    )
    doubled_grad = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
        grad_gate * 2, grad_up * 2, gate, up, indices, offsets, qtype, k
    )
    torch.testing.assert_close(doubled_grad, pair_grad * 2, rtol=0, atol=0)

    rng = np.random.default_rng(3)
    sample = _sample_rows(offsets.cpu().numpy(), rng)
    expert_of_group = indices.cpu().numpy()
    gate_host, up_host = {}, {}
    noise = forward_noise(qtype, x.shape[0], n, 2)
    for group, row in sample:
        expert = int(expert_of_group[group])
        if expert not in gate_host:
            gate_host[expert] = gate[expert].cpu().numpy()
            up_host[expert] = up[expert].cpu().numpy()
        x_row = bits(x[row:row + 1])
        assert_matches_f32_reference(out_gate[row:row + 1], oracle.mmq_forward(qtype, x_row, gate_host[expert], n, k), noise)
        assert_matches_f32_reference(out_up[row:row + 1], oracle.mmq_forward(qtype, x_row, up_host[expert], n, k), noise)
        expected = oracle.grad_input(qtype, bits(grad_gate[row:row + 1]), gate_host[expert], n, k).astype(np.float64)
        expected += oracle.grad_input(qtype, bits(grad_up[row:row + 1]), up_host[expert], n, k)
        assert_matches_f32_reference(pair_grad[row:row + 1], expected.astype(np.float32), accumulate_noise=2e-6)


def test_down_projection_at_its_configured_size(ops, oracle):
    """256 experts, Q4_K [2048, 512], 4096 tokens x top-8 skewed routing (32 768 rows), forward only."""
    tgo, synth = ops
    qtype, n, k, experts = QTYPES["Q4_K"], 2048, 512, 256
    token_of_row, indices, offsets, _ = synth.zipf_routing(4096, experts, 8, 11, device="cuda")
    rows = token_of_row.numel()
    generator = torch.Generator(device="cuda").manual_seed(8)
    x = torch.randn(rows, k, device="cuda", generator=generator).to(torch.bfloat16)
    down = synth.random_packed_weight(qtype, (experts, n), k, 73, device="cuda")
    out = tgo.grouped_mmq(x, down, indices, offsets, qtype, n)
    torch.testing.assert_close(tgo.grouped_mmq(x * 2, down, indices, offsets, qtype, n), out * 2, rtol=0, atol=0)
    flip = _reverse_within_groups(offsets.cpu().numpy(), rows)
    flipped = tgo.grouped_mmq(x.index_select(0, flip), down, indices, offsets, qtype, n)
    torch.testing.assert_close(flipped, out.index_select(0, flip), rtol=0, atol=0)
    expert_of_group = indices.cpu().numpy()
    for group, row in _sample_rows(offsets.cpu().numpy(), np.random.default_rng(4), per_kind=4):
        host = down[int(expert_of_group[group])].cpu().numpy()
        assert_matches_f32_reference(out[row:row + 1], oracle.mmq_forward(qtype, bits(x[row:row + 1]), host, n, k), forward_noise(qtype, x.shape[0], n))


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_dense_at_its_largest_configured_size(ops, oracle, qname):
    """M = 4096, N = 4096, K = 2048 for every format: homogeneity everywhere, the oracle on eight rows."""
    tgo, synth = ops
    qtype, m, n, k = QTYPES[qname], 4096, 4096, 2048
    host = synth.random_packed_weight(qtype, (n,), k, seed=500 + qtype)
    weight = host.cuda()
    generator = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(m, k, device="cuda", generator=generator).to(torch.bfloat16)
    dy = torch.randn(m, n, device="cuda", generator=generator).to(torch.bfloat16)
    out = tgo.mmq(x, weight, qtype, n)
    grad = torch.ops.torch_ggml_ops.mmq_grad_input.default(dy, weight, qtype, k)
    torch.testing.assert_close(tgo.mmq(x * 2, weight, qtype, n), out * 2, rtol=0, atol=0)
    torch.testing.assert_close(torch.ops.torch_ggml_ops.mmq_grad_input.default(dy * 2, weight, qtype, k), grad * 2, rtol=0, atol=0)
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 2049, 4095], device="cuda")
    packed = host.numpy()
    assert_matches_f32_reference(out.index_select(0, rows), oracle.mmq_forward(qtype, bits(x.index_select(0, rows)), packed, n, k),
                                 forward_noise(qtype, x.shape[0], n))
    assert_matches_f32_reference(
        grad.index_select(0, rows), oracle.grad_input(qtype, bits(dy.index_select(0, rows)), packed, n, k),
        accumulate_noise=2e-6,
    )


@pytest.mark.parametrize("tokens", (1, 4, 8))
def test_decode_configuration_against_the_oracle(ops, oracle, tokens):
    """T tokens x top-8 over 256 experts: gate+up pair IQ2_S [512, 2048], down Q6_K [2048, 512], and the dense
    Q3_K [4096, 2048] single-row projection; small enough for the oracle to cover every row."""
    tgo, synth = ops
    experts = 256
    token_of_row, indices, offsets, _ = synth.zipf_routing(tokens, experts, 8, 100 * tokens, device="cuda")
    rows = token_of_row.numel()
    assert tgo._native.lib.tgo_forward_kernel_family(rows, indices.numel()) == b"gemv"  # the decode kernel family
    gate_host = synth.random_packed_weight(QTYPES["IQ2_S"], (experts, 512), 2048, seed=81)
    up_host = synth.random_packed_weight(QTYPES["IQ2_S"], (experts, 512), 2048, seed=82)
    down_host = synth.random_packed_weight(QTYPES["Q6_K"], (experts, 2048), 512, seed=83)
    generator = torch.Generator(device="cuda").manual_seed(tokens)
    hidden = torch.randn(tokens, 2048, device="cuda", generator=generator).to(torch.bfloat16)
    x = hidden.index_select(0, token_of_row).contiguous()
    middle = torch.randn(rows, 512, device="cuda", generator=generator).to(torch.bfloat16)
    out_gate, out_up = tgo.grouped_mmq_pair(x, gate_host.cuda(), up_host.cuda(), indices, offsets, QTYPES["IQ2_S"], 512)
    out_down = tgo.grouped_mmq(middle, down_host.cuda(), indices, offsets, QTYPES["Q6_K"], 2048)
    group_experts, group_ends = indices.tolist(), offsets.tolist()
    for out, host in ((out_gate, gate_host), (out_up, up_host)):
        exact = oracle.grouped(oracle.mmq_forward, QTYPES["IQ2_S"], bits(x), host.numpy(), group_experts, group_ends, 512, 2048, 512)
        assert_matches_f32_reference(out, exact)
    exact = oracle.grouped(oracle.mmq_forward, QTYPES["Q6_K"], bits(middle), down_host.numpy(), group_experts, group_ends, 2048, 512, 2048)
    assert_matches_f32_reference(out_down, exact)

    dense_host = synth.random_packed_weight(QTYPES["Q3_K"], (4096,), 2048, seed=84)
    single = hidden[:1].contiguous()
    dense_out = tgo.mmq(single, dense_host.cuda(), QTYPES["Q3_K"], 4096)
    assert_matches_f32_reference(dense_out, oracle.mmq_forward(QTYPES["Q3_K"], bits(single), dense_host.numpy(), 4096, 2048))
