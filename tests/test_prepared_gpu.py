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

from helpers import OPERAND_NOISE, QTYPES, assert_matches_f32_reference, bits, random_bf16

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


@pytest.mark.parametrize("kind", ("int8", "half", "scaled"))
def test_workspace_of_a_named_kind_matches_the_oracle(ops, oracle, kind):
    """A caller may name the operand kind of a workspace: every format's kernel of that kind reads it."""
    tgo, synth = ops
    rows, k = 300, 1024
    x = random_bf16((rows, k), seed=17)
    workspace = tgo.quantize_q8_1(x, operand=kind)
    for qname, n in (("Q4_K", 96), ("Q6_K", 37), ("IQ2_S", 160), ("Q5_K", 512), ("Q3_K", 64)):
        qtype = QTYPES[qname]
        host = synth.random_packed_weight(qtype, (n,), k, seed=900 + qtype)
        prepared = tgo.mmq_prepared(workspace, host.cuda(), rows, k, qtype, n, operand=kind)
        assert_matches_f32_reference(prepared, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k),
                                     accumulate_noise=OPERAND_NOISE[kind])
    # the same workspace read as another kind: refused on the device, every output NaN
    other = "int8" if kind != "int8" else "scaled"
    weight = synth.random_packed_weight(12, (64,), k, seed=5).cuda()
    assert torch.isnan(tgo.mmq_prepared(workspace, weight, rows, k, 12, 64, operand=other).float()).all()
    with pytest.raises(ValueError, match="operand must be"):
        tgo.quantize_q8_1(x, operand="fp8")


def test_multi_projection_of_a_long_sequence_takes_the_scaled_kernels(ops):
    """q/k/v of 2048 rows fill the chip together: mmq_multi quantizes for, and runs, the scaled kernels, and each
    projection agrees with a separate mmq (scaled or int8 by its own size) within the scaled kind's rounding."""
    from torch_ggml_ops import prepared

    tgo, synth = ops
    rows, k, widths = 2048, 512, (2048, 1024, 1024)
    qtypes = [QTYPES["Q4_K"], QTYPES["Q4_K"], QTYPES["Q6_K"]]
    assert prepared.multi_operand(qtypes, rows, widths) == "scaled"
    assert prepared.multi_operand(qtypes, 40, widths) == "int8"
    assert prepared.multi_operand([QTYPES["IQ2_S"]] * 2, 40, widths[:2]) == "half"
    assert prepared.multi_operand([QTYPES["IQ2_S"], QTYPES["Q4_K"]], 40, widths[:2]) == "int8"
    weights = [synth.random_packed_weight(q, (n,), k, seed=60 + i).cuda() for i, (q, n) in enumerate(zip(qtypes, widths))]
    x = random_bf16((rows, k), seed=9)
    outputs = tgo.mmq_multi(x, weights, qtypes, widths)
    for output, weight, qtype, n in zip(outputs, weights, qtypes, widths):
        plain = tgo.mmq(x, weight, qtype, n).float()
        tolerance = plain.abs() * 2.0**-7 + 2 * OPERAND_NOISE["scaled"] * float(plain.abs().max())
        assert bool(((output.float() - plain).abs() <= tolerance).all())


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
