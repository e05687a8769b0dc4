"""GPU parity of the prepared-activation operators (-m gpu): quantize once, several projections.

The reference has no such operator, so the oracle here is the library's own ``mmq`` (which the
other tests pin against the CPU oracle): ``mmq_prepared`` must reproduce it bit for bit, and
``mmq_multi``'s gradient must equal the sum of the projections' ``mmq_grad_input``.

A workspace that is quantized before its weight format is known holds int8 tiles and runs the int8 kernels,
while ``mmq`` by default multiplies fp16 operands for IQ2_S: bit-for-bit equality therefore holds with the
int8 operands forced (and by default for the other formats); under the default the two agree up to fp32 rounding.
"""

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


@pytest.fixture(params=("auto", "int8"))
def operand(request):
    from torch_ggml_ops import _native

    _native.set_forward_operand(request.param)
    yield request.param
    _native.set_forward_operand("auto")


def _assert_same(operand, qname, actual, expected):
    if operand == "int8" or qname != "IQ2_S":
        torch.testing.assert_close(actual, expected, rtol=0, atol=0)
    else:   # one bf16 ulp where the fp32 sums round differently
        torch.testing.assert_close(actual.detach().float(), expected.detach().float(), rtol=2.0**-7,
                                   atol=1e-5 * float(expected.detach().float().abs().max()))


@pytest.mark.parametrize("rows", (1, 5, 77, 300))
def test_prepared_equals_mmq_bit_for_bit(ops, oracle, operand, rows):
    tgo, synth = ops
    k = 1024
    x = random_bf16((rows, k), seed=rows)
    workspace = tgo.quantize_q8_1(x)
    assert workspace.dtype == torch.uint8 and workspace.is_cuda
    for qname, n in (("Q4_K", 96), ("Q6_K", 37), ("IQ2_S", 160), ("Q5_K", 512), ("Q3_K", 64)):
        qtype = QTYPES[qname]
        host = synth.random_packed_weight(qtype, (n,), k, seed=700 + qtype)
        weight = host.cuda()
        prepared = tgo.mmq_prepared(workspace, weight, rows, k, qtype, n)
        _assert_same(operand, qname, prepared, tgo.mmq(x, weight, qtype, n))
        assert_matches_f32_reference(prepared, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k))


def test_multi_projection_forward_and_gradient(ops, operand):
    tgo, synth = ops
    k, shapes = 512, (("Q4_K", 256), ("Q5_K", 64), ("Q6_K", 64))
    weights = [synth.random_packed_weight(QTYPES[q], (n,), k, seed=800 + i).cuda() for i, (q, n) in enumerate(shapes)]
    qtypes = [QTYPES[q] for q, _ in shapes]
    widths = [n for _, n in shapes]
    x = random_bf16((3, 40, k), seed=31).requires_grad_(True)
    outputs = tgo.mmq_multi(x, weights, qtypes, widths)
    grads = [random_bf16((3, 40, n), seed=40 + i) for i, n in enumerate(widths)]
    torch.autograd.backward(outputs, grads)

    y = x.detach().clone().requires_grad_(True)
    separate = [tgo.mmq(y, w, q, n) for w, q, n in zip(weights, qtypes, widths)]
    for fused, plain, (qname, _) in zip(outputs, separate, shapes):
        assert fused.shape == plain.shape
        _assert_same(operand, qname, fused, plain)
    expected = None
    for grad, weight, qtype in zip(grads, weights, qtypes):
        term = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad, weight, qtype, k)
        expected = term if expected is None else expected + term
    torch.testing.assert_close(x.grad, expected, rtol=0, atol=0)

    # a projection whose output is unused contributes nothing
    z = x.detach().clone().requires_grad_(True)
    first, _, _ = tgo.mmq_multi(z, weights, qtypes, widths)
    first.backward(grads[0])
    only = torch.ops.torch_ggml_ops.mmq_grad_input.default(grads[0], weights[0], qtypes[0], k)
    torch.testing.assert_close(z.grad, only, rtol=0, atol=0)


def test_prepared_rejects_mismatched_workspace(ops):
    tgo, synth = ops
    x = random_bf16((8, 512), seed=1)
    workspace = tgo.quantize_q8_1(x)
    weight = synth.random_packed_weight(12, (32,), 512, seed=2).cuda()
    with pytest.raises(RuntimeError, match="workspace holds"):
        tgo.mmq_prepared(workspace, weight, 64, 512, 12, 32)
    with pytest.raises(RuntimeError, match="packed_weight has"):
        tgo.mmq_prepared(workspace, weight, 8, 512, 13, 32)
    with pytest.raises(RuntimeError, match="multiple of 256"):
        tgo.quantize_q8_1(random_bf16((4, 100), seed=3))
