"""GPU parity of the gathered grouped operators (-m gpu): token -> sorted-row gather inside the quantizer.

The reference takes pre-sorted rows, so the oracle is the library's own grouped operator on
``hidden.index_select(0, row_index)`` (pinned against the CPU oracle by the other tests): forward
results must agree bit for bit, and the gradient with respect to the token activations must equal
the per-token fp32 sum of the sorted rows' grad-input.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits, random_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


def _routing(tokens, top_k, experts, seed):
    """Top-k routing of ``tokens`` tokens: (row_index sorted by expert, active experts, inclusive offsets)."""
    generator = np.random.default_rng(seed)
    chosen = np.stack([generator.permutation(experts)[:top_k] for _ in range(tokens)])
    flat_expert = chosen.reshape(-1)
    flat_token = np.repeat(np.arange(tokens), top_k)
    order = np.argsort(flat_expert, kind="stable")
    counts = np.bincount(flat_expert, minlength=experts)
    active = np.nonzero(counts)[0]
    return (
        torch.from_numpy(flat_token[order]).cuda(),
        torch.from_numpy(active.astype(np.int64)).cuda(),
        torch.from_numpy(np.cumsum(counts[active]).astype(np.int32)).cuda(),
    )


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize("tokens,top_k", ((3, 2), (97, 4)))
def test_gathered_pair_equals_index_select(ops, oracle, qname, tokens, top_k):
    tgo, synth = ops
    qtype, n, k, experts = QTYPES[qname], 96, 1024, 8
    host_first = synth.random_packed_weight(qtype, (experts, n), k, seed=900 + qtype)
    host_second = synth.random_packed_weight(qtype, (experts, n), k, seed=910 + qtype)
    first, second = host_first.cuda(), host_second.cuda()
    hidden = random_bf16((tokens, k), seed=tokens)
    row_index, indices, offsets = _routing(tokens, top_k, experts, seed=tokens + top_k)
    sorted_rows = hidden.index_select(0, row_index)

    gathered = tgo.grouped_mmq_pair_gathered(hidden, row_index, first, second, indices, offsets, qtype, n)
    plain = tgo.grouped_mmq_pair(sorted_rows, first, second, indices, offsets, qtype, n)
    for a, b in zip(gathered, plain):
        assert a.shape == (tokens * top_k, n)
        torch.testing.assert_close(a, b, rtol=0, atol=0)
    single = tgo.grouped_mmq_gathered(hidden, row_index, second, indices, offsets, qtype, n)
    torch.testing.assert_close(single, plain[1], rtol=0, atol=0)
    exact = oracle.grouped(
        oracle.mmq_forward, qtype, bits(sorted_rows), host_first.numpy(), indices.tolist(), offsets.tolist(), n, k, n
    )
    assert_matches_f32_reference(gathered[0], exact)


def test_gathered_gradient_sums_rows_per_token(ops):
    tgo, synth = ops
    qtype, n, k, experts, tokens, top_k = 13, 128, 512, 6, 50, 3
    first = synth.random_packed_weight(qtype, (experts, n), k, seed=21).cuda()
    second = synth.random_packed_weight(qtype, (experts, n), k, seed=22).cuda()
    row_index, indices, offsets = _routing(tokens, top_k, experts, seed=9)
    rows = tokens * top_k
    grad_first = random_bf16((rows, n), seed=23)
    grad_second = random_bf16((rows, n), seed=24)

    hidden = random_bf16((tokens, k), seed=20).requires_grad_(True)
    outputs = tgo.grouped_mmq_pair_gathered(hidden, row_index, first, second, indices, offsets, qtype, n)
    torch.autograd.backward(outputs, (grad_first, grad_second))
    grad_rows = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
        grad_first, grad_second, first, second, indices, offsets, qtype, k
    )
    expected = torch.zeros((tokens, k), dtype=torch.float64, device="cuda")
    expected.index_add_(0, row_index, grad_rows.double())
    # fp32 accumulation of at most top_k bf16 terms, one rounding to bf16
    torch.testing.assert_close(hidden.grad.double(), expected, rtol=2**-8, atol=1e-30)

    single = random_bf16((tokens, k), seed=20).requires_grad_(True)
    tgo.grouped_mmq_gathered(single, row_index, first, indices, offsets, qtype, n).backward(grad_first)
    rows_only = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad_first, first, indices, offsets, qtype, k)
    expected = torch.zeros((tokens, k), dtype=torch.float64, device="cuda")
    expected.index_add_(0, row_index, rows_only.double())
    torch.testing.assert_close(single.grad.double(), expected, rtol=2**-8, atol=1e-30)


def test_gathered_index_outside_the_input_reads_zeros(ops):
    """The C entry point treats an index outside the token range as a row of zeros (output exactly zero)."""
    tgo, synth = ops
    qtype, n, k = 12, 64, 512
    weight = synth.random_packed_weight(qtype, (2, n), k, seed=31).cuda()
    hidden = random_bf16((4, k), seed=32)
    row_index = torch.tensor([2, -1, 0, 9, 3], device="cuda", dtype=torch.int64)
    indices = torch.tensor([0, 1], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([2, 5], device="cuda", dtype=torch.int32)
    out = tgo.grouped_mmq_gathered(hidden, row_index, weight, indices, offsets, qtype, n)
    padded = torch.cat([hidden, torch.zeros_like(hidden[:1])])
    safe = torch.tensor([2, 4, 0, 4, 3], device="cuda")
    expected = tgo.grouped_mmq(padded.index_select(0, safe), weight, indices, offsets, qtype, n)
    torch.testing.assert_close(out, expected, rtol=0, atol=0)
    assert torch.count_nonzero(out[1]) == 0 and torch.count_nonzero(out[3]) == 0


def test_gathered_gradient_skips_rows_outside_the_input(ops):
    """Backward through an index with entries outside the token range (dropped tokens): those rows add nothing,
    the others sum per token as usual, and a second backward returns the same bits."""
    tgo, synth = ops
    qtype, n, k = 12, 64, 512
    weight = synth.random_packed_weight(qtype, (2, n), k, seed=51).cuda()
    row_index = torch.tensor([2, -1, 0, 9, 3, 2], device="cuda", dtype=torch.int64)
    indices = torch.tensor([0, 1], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([2, 6], device="cuda", dtype=torch.int32)
    grad_output = random_bf16((6, n), seed=53)
    grads = []
    for _ in range(2):
        hidden = random_bf16((4, k), seed=52).requires_grad_(True)
        tgo.grouped_mmq_gathered(hidden, row_index, weight, indices, offsets, qtype, n).backward(grad_output)
        grads.append(hidden.grad)
    torch.testing.assert_close(grads[0], grads[1], rtol=0, atol=0)
    grad_rows = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad_output, weight, indices, offsets, qtype, k)
    expected = torch.zeros((4, k), dtype=torch.float64, device="cuda")
    for row, token in enumerate(row_index.tolist()):
        if 0 <= token < 4:
            expected[token] += grad_rows[row].double()
    torch.testing.assert_close(grads[0].double(), expected, rtol=2**-8, atol=1e-30)
    assert torch.count_nonzero(grads[0][1]) == 0   # token 1 has no row


def test_gathered_rejects_bad_index(ops):
    tgo, synth = ops
    weight = synth.random_packed_weight(12, (2, 32), 256, seed=41).cuda()
    hidden = random_bf16((4, 256), seed=42)
    indices = torch.tensor([0], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([4], device="cuda", dtype=torch.int32)
    with pytest.raises(RuntimeError, match="row_index must have dtype torch.int64"):
        tgo.grouped_mmq_gathered(hidden, torch.arange(4, device="cuda", dtype=torch.int32), weight, indices, offsets, 12, 32)
    with pytest.raises(RuntimeError, match="one-dimensional"):
        tgo.grouped_mmq_gathered(hidden, torch.zeros((2, 2), device="cuda", dtype=torch.int64), weight, indices, offsets, 12, 32)


@pytest.mark.parametrize("tokens,rows,features", ((5, 23, 256), (97, 388, 2048), (300, 64, 2304)))
def test_rows_to_tokens_kernel_equals_an_ordered_index_put(ops, tokens, rows, features):
    """The scatter of the gathered operators' backward (tgo_rows_to_tokens over a stable sort of the gather index)
    against index_put_(accumulate=True) on fp32 copies, which also adds each token's rows in row order: the same bits.
    Some rows name no token (dropped), some tokens have no row (zeros)."""
    from torch_ggml_ops import gathered

    generator = torch.Generator(device="cuda").manual_seed(tokens + rows)
    grad_rows = torch.randn(rows, features, device="cuda", generator=generator).to(torch.bfloat16)
    row_index = torch.randint(0, tokens, (rows,), device="cuda", generator=generator)
    row_index[::7] = -1
    row_index[3::11] = tokens + 5
    actual = gathered._scatter_to_tokens(grad_rows, row_index, tokens)
    present = (row_index >= 0) & (row_index < tokens)
    total = torch.zeros((tokens, features), dtype=torch.float32, device="cuda")
    total.index_put_((row_index.clamp(0, tokens - 1),), grad_rows.float() * present.unsqueeze(1), accumulate=True)
    assert actual.shape == (tokens, features) and actual.dtype == torch.bfloat16
    torch.testing.assert_close(actual, total.to(torch.bfloat16), rtol=0, atol=0)
