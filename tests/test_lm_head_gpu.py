"""The chunked LM-head loss against the unchunked computation (-m gpu).

`chunked_lm_head_loss` walks the rows in chunks (the reference's production schedule,
docs/mmq_fwd_optimization.md:293) and must give the loss and the hidden-state gradient of
`cross_entropy(mmq(hidden, W).float(), targets)`: the loss up to fp32 summation order, the gradient up to the
bf16 rounding of the logit gradients that both paths hand to `mmq_grad_input`.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, bits, f32, nrmse, random_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


@pytest.mark.parametrize("qname,chunk", [("Q6_K", 128), ("Q6_K", 64), ("Q4_K", 256)])
def test_chunked_loss_equals_the_unchunked_computation(ops, oracle, qname, chunk):
    tgo, synth = ops
    qtype, rows, k, vocabulary = QTYPES[qname], 300, 512, 1000   # ragged last chunk, vocabulary not a tile multiple
    host = synth.random_packed_weight(qtype, (vocabulary,), k, seed=880 + qtype, scale_range=(1e-3, 3e-2))
    weight = host.cuda()
    generator = torch.Generator().manual_seed(88)
    targets = torch.randint(0, vocabulary, (rows,), generator=generator).cuda()
    targets[5] = -100
    targets[299] = -100

    hidden = random_bf16((rows, k), seed=881).requires_grad_(True)
    loss = tgo.chunked_lm_head_loss(hidden, weight, targets, qtype, vocabulary, chunk_rows=chunk)
    (loss * 3.0).backward()

    reference_hidden = random_bf16((rows, k), seed=881).requires_grad_(True)
    logits = tgo.mmq(reference_hidden, weight, qtype, vocabulary)
    reference = torch.nn.functional.cross_entropy(logits.float(), targets, ignore_index=-100)
    (reference * 3.0).backward()

    assert loss.dtype == torch.float32 and loss.dim() == 0
    torch.testing.assert_close(loss, reference, rtol=1e-5, atol=1e-6)
    # (two bf16 roundings separate the paths: the logit gradients, and the scaling by the incoming gradient)
    assert nrmse(f32(hidden.grad), f32(reference_hidden.grad)) < 5e-3
    assert not f32(hidden.grad)[5].any() and not f32(hidden.grad)[299].any()   # ignored rows get no gradient

    # and against the oracle's exact evaluation of the same q8_1 algebra on a few rows
    sample = [0, 127, 128, 298]
    exact_logits = oracle.mmq_forward(qtype, bits(hidden.detach()[sample]), host.numpy(), vocabulary, k).astype(np.float64)
    exact = -(exact_logits - np.log(np.exp(exact_logits - exact_logits.max(1, keepdims=True)).sum(1, keepdims=True))
              - exact_logits.max(1, keepdims=True))[np.arange(len(sample)), targets[sample].cpu().numpy()]
    per_row = torch.nn.functional.cross_entropy(logits.detach().float()[sample], targets[sample], reduction="none")
    np.testing.assert_allclose(per_row.cpu().numpy(), exact, rtol=0, atol=2e-2 * np.abs(exact_logits).max())


def test_chunked_loss_without_gradient_and_bad_arguments(ops):
    tgo, synth = ops
    weight = synth.random_packed_weight(12, (64,), 256, seed=889).cuda()
    hidden = random_bf16((10, 256), seed=890)
    targets = torch.zeros(10, dtype=torch.int64, device="cuda")
    with torch.no_grad():
        loss = tgo.chunked_lm_head_loss(hidden, weight, targets, 12, 64, chunk_rows=4)
    assert torch.isfinite(loss)
    with pytest.raises(RuntimeError, match="one entry per row"):
        tgo.chunked_lm_head_loss(hidden, weight, targets[:5], 12, 64)
    with pytest.raises(RuntimeError, match="chunk_rows"):
        tgo.chunked_lm_head_loss(hidden, weight, targets, 12, 64, chunk_rows=0)
