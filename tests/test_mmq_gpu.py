"""GPU parity of the dense operators against the CPU oracle (run with -m gpu).

Mirrors the reference's tests/test_mmq.py with seeded synthetic blocks in place of its
checkpoint: forward error against the dequantize-then-matmul path, one-hot and random
cotangents for the grad-input operator, stream semantics, opcheck/compile and the
fail-fast error contract.  Everything goes through the registered operators, i.e.
through the C ABI of libtgo_hip.so.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits, f32, max_rel_to_peak, nrmse, random_bf16

pytestmark = pytest.mark.gpu

# forward tolerance against x @ bf16(W)^T: q8_1 rounding of the activations costs about 0.6 % of the
# output norm; the stated bound is 1e-2, measured on norms (NRMSE and max error over max reference)
FORWARD_TOLERANCE = 1e-2


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth
    from torch_ggml_ops import _native

    assert torch.cuda.is_available()
    return torch_ggml_ops, _native, synth


def _weight(synth, qtype, n, k, seed):
    host = synth.random_packed_weight(qtype, (n,), k, seed=seed)
    return host, host.cuda()


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_dequant_kernel_is_bit_exact(ops, oracle, qname):
    _, native, synth = ops
    qtype = QTYPES[qname]
    for rows, k in ((37, 2048), (5, 256), (130, 512)):
        host, device = _weight(synth, qtype, rows, k, seed=100 + qtype + rows)
        out = torch.empty(rows, k, dtype=torch.bfloat16, device="cuda")
        native.check(native.lib.tgo_dequant_bf16(device.data_ptr(), out.data_ptr(), rows, k, qtype, None))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bits(out), oracle.dequant_bf16(qtype, host.numpy(), k))


def test_dequant_kernel_handles_signed_and_subnormal_scales(ops, oracle):
    _, native, _ = ops
    rng = np.random.default_rng(99)
    for qname, qtype in QTYPES.items():
        block = native.lib.tgo_block_bytes(qtype)
        rows, k = 24, 512
        data = rng.integers(0, 256, (rows * 2, block), dtype=np.uint8)
        offsets = {11: (108,), 12: (0, 2), 13: (0, 2), 14: (208,), 22: (0,)}[qtype]
        for offset in offsets:
            raw = (
                (rng.integers(0, 2, rows * 2).astype(np.uint16) << 15)
                | (rng.integers(0, 31, rows * 2).astype(np.uint16) << 10)  # exponent 0 = subnormal
                | rng.integers(0, 1024, rows * 2).astype(np.uint16)
            )
            data[:, offset : offset + 2] = raw.view(np.uint8).reshape(-1, 2)
        host = data.reshape(rows, -1)
        device = torch.from_numpy(host).cuda()
        out = torch.empty(rows, k, dtype=torch.bfloat16, device="cuda")
        native.check(native.lib.tgo_dequant_bf16(device.data_ptr(), out.data_ptr(), rows, k, qtype, None))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bits(out), oracle.dequant_bf16(qtype, host, k), err_msg=qname)


@pytest.mark.parametrize("rows", (48, 300))
@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_grad_input_decoders_handle_signed_and_subnormal_scales(ops, oracle, qname, rows):
    """The dequantizers inside the grad-input kernels (their own code, not the dequant kernel's): random block bytes
    with negative and subnormal fp16 super-scales, identity cotangents, so that row i of the result is weight row i
    as the reference decoder rounds it (compared as numbers: a product's zeros lose their sign in the accumulation).
    48 rows: the short-task kernels; 300: the others."""
    _, native, _ = ops
    qtype, n, k = QTYPES[qname], rows, 512
    rng = np.random.default_rng(1234 + qtype + rows)
    block = native.lib.tgo_block_bytes(qtype)
    data = rng.integers(0, 256, (n * (k // 256), block), dtype=np.uint8)
    for offset in {11: (108,), 12: (0, 2), 13: (0, 2), 14: (208,), 22: (0,)}[qtype]:
        raw = (
            (rng.integers(0, 2, len(data)).astype(np.uint16) << 15)
            | (rng.integers(0, 31, len(data)).astype(np.uint16) << 10)   # exponent 0 = subnormal
            | rng.integers(0, 1024, len(data)).astype(np.uint16)
        )
        data[:, offset : offset + 2] = raw.view(np.uint8).reshape(-1, 2)
    host = data.reshape(n, -1)
    identity = torch.eye(n, device="cuda", dtype=torch.bfloat16)
    actual = torch.ops.torch_ggml_ops.mmq_grad_input.default(identity, torch.from_numpy(host).cuda(), qtype, k)
    logical = oracle.bf16_to_f32(oracle.dequant_bf16(qtype, host, k))
    np.testing.assert_array_equal(f32(actual), logical)
    # the grouped operator takes other kernels (role-split / pipelined / short-task) than the dense one
    experts = torch.tensor([0], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([n], device="cuda", dtype=torch.int32)
    grouped = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(
        identity, torch.from_numpy(host).cuda().unsqueeze(0), experts, offsets, qtype, k)
    np.testing.assert_array_equal(f32(grouped), logical)


@pytest.mark.parametrize("rows,k", [(1, 256), (33, 512), (129, 2048)])
def test_q8_1_quantizer_matches_oracle_bit_for_bit(ops, oracle, rows, k):
    _, native, _ = ops
    x = random_bf16((rows, k), seed=7 + rows, scale=2.0)
    x[0, :32] = 0  # a zero block
    # exact halves (scale 127/amax = 1): roundf sends them away from zero; and values that round to -0
    x[0, 32:64] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 126.5, -126.5, -0.25, 0.25, -0.0, 3.5, -3.5] * 2)
    workspace = torch.empty(native.lib.tgo_q8_workspace_bytes(rows, k), dtype=torch.uint8, device="cuda")
    native.check(native.lib.tgo_quantize_q8_1(x.data_ptr(), workspace.data_ptr(), rows, k, None))
    q = torch.empty(rows, k, dtype=torch.int8, device="cuda")
    d = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    s = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    native.check(
        native.lib.tgo_q8_workspace_unpack(workspace.data_ptr(), q.data_ptr(), d.data_ptr(), s.data_ptr(), rows, k, None)
    )
    torch.cuda.synchronize()
    q_ref, d_ref, s_ref = oracle.quantize_q8_1(bits(x))
    np.testing.assert_array_equal(q.cpu().numpy(), q_ref)
    np.testing.assert_array_equal(d.cpu().numpy().view(np.uint32), d_ref.view(np.uint32))
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))


@pytest.mark.parametrize("kind", (0, 1))   # TGO_OPERAND_INT8, TGO_OPERAND_HALF: both keep the quants themselves
def test_q8_1_quantizer_matches_oracle_for_every_amax(ops, oracle, kind):
    """Activations are bf16, so a block's amax is one of 2^15 values: every one between 2^-100 and 2^100 (and zero)
    heads a block here, followed by 31 fractions of it of both signs, and quants, scales (d = amax / 127, with
    127 / amax behind the quants) and sums must equal the oracle's bit for bit."""
    _, native, _ = ops
    exponents = np.arange(127 - 100, 127 + 101, dtype=np.uint32)
    amax_bits = np.concatenate([[0], ((exponents[:, None] << 7) | np.arange(128, dtype=np.uint32)[None, :]).reshape(-1)])
    blocks = amax_bits.size
    rows = (blocks + 63) // 64
    amax_bits = np.concatenate([amax_bits, np.full(rows * 64 - blocks, 0x3F80, dtype=np.uint32)])
    amax = torch.from_numpy((amax_bits << 16).astype(np.uint32).view(np.float32).copy()).cuda()
    generator = torch.Generator(device="cuda").manual_seed(5)
    factors = torch.rand(rows * 64, 32, device="cuda", generator=generator) * 2.0 - 1.0
    factors[:, 0] = 1.0
    factors[:, 1] = -1.0
    factors[:, 2:10] = torch.tensor([0.5, -0.5, 1.5 / 127, 2.5 / 127, -63.5 / 127, 126.5 / 127, 0.0, -0.0], device="cuda")
    x = (amax[:, None] * factors).to(torch.bfloat16).reshape(rows, 2048).contiguous()
    k = 2048
    workspace = torch.empty(native.lib.tgo_q8_workspace_bytes(rows, k), dtype=torch.uint8, device="cuda")
    native.check(native.lib.tgo_quantize_q8_1_as(x.data_ptr(), workspace.data_ptr(), rows, k, kind, None))
    q = torch.empty(rows, k, dtype=torch.int8, device="cuda")
    d = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    s = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    native.check(
        native.lib.tgo_q8_workspace_unpack(workspace.data_ptr(), q.data_ptr(), d.data_ptr(), s.data_ptr(), rows, k, None)
    )
    torch.cuda.synchronize()
    q_ref, d_ref, s_ref = oracle.quantize_q8_1(bits(x))
    np.testing.assert_array_equal(d.cpu().numpy().view(np.uint32), d_ref.view(np.uint32))
    np.testing.assert_array_equal(q.cpu().numpy(), q_ref)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize("shape,n", [((3, 43), 37), ((1,), 64), ((16,), 130), ((300,), 96)])
def test_forward_matches_oracle(ops, oracle, qname, shape, n):
    tgo, _, synth = ops
    qtype, k = QTYPES[qname], 2048
    host, device = _weight(synth, qtype, n, k, seed=1234 + qtype)
    x = random_bf16((*shape, k), seed=1234)
    actual = tgo.mmq(x, device, qtype, n)
    assert actual.shape == (*shape, n) and actual.dtype == torch.bfloat16 and actual.is_contiguous()
    assert torch.isfinite(actual).all()
    flat = bits(x).reshape(-1, k)
    # same algebra, float64 accumulation: differs only by fp32 summation and the final rounding
    assert_matches_f32_reference(actual.reshape(-1, n), oracle.mmq_forward(qtype, flat, host.numpy(), n, k))
    # the dequantize-then-matmul path, within the stated tolerance
    expected = oracle.linear_forward(qtype, flat, host.numpy(), n, k)
    assert nrmse(f32(actual).reshape(-1, n), expected) < FORWARD_TOLERANCE
    if flat.shape[0] * n >= 1024:
        assert max_rel_to_peak(f32(actual).reshape(-1, n), expected) < FORWARD_TOLERANCE


@pytest.mark.parametrize("qname", ("Q4_K", "Q5_K"))
def test_forward_distance_from_the_fp16_scale_numerics(ops, oracle, qname):
    """For Q4_K / Q5_K the reference stores four per-block scale values as fp16 (weights: d*sc and -dmin*m,
    csrc/vendor/llama_cpp/mmq-load-targets.cuh:190-195; activations: d and sum, csrc/mmq_core.cuh:202-203); this
    library keeps them in fp32.  The distance between its output and the oracle's half-scale mode is bounded here:
    it is the bf16 rounding of the output (up to 2^-9 of an element, 1.1e-3 on norms) plus a few 1e-4 from the fp16 scales."""
    tgo, _, synth = ops
    qtype, rows, n, k = QTYPES[qname], 300, 96, 2048
    host, device = _weight(synth, qtype, n, k, seed=8642 + qtype)
    x = random_bf16((rows, k), seed=8642)
    actual = f32(tgo.mmq(x, device, qtype, n))
    half_mode = oracle.mmq_forward_half_scales(qtype, bits(x), host.numpy(), n, k)
    fp32_mode = oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k)
    distance, peak = nrmse(actual, half_mode), max_rel_to_peak(actual, half_mode)
    between_modes = nrmse(fp32_mode, half_mode)
    print(f"{qname}: library vs half-scale oracle NRMSE {distance:.2e}, max/peak {peak:.2e}; fp32 vs half-scale oracle {between_modes:.2e}")
    assert between_modes < 5e-4
    assert distance < 3e-3 and peak < 5e-3


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_grad_input_decodes_every_logical_weight_value(ops, oracle, qname):
    _, _, synth = ops
    qtype = QTYPES[qname]
    host, device = _weight(synth, qtype, 37, 2048, seed=77 + qtype)
    grad_output = torch.zeros(1, 37, device="cuda", dtype=torch.bfloat16)
    grad_output[0, 17] = 1
    actual = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad_output, device, qtype, 2048)
    logical = oracle.bf16_to_f32(oracle.dequant_bf16(qtype, host.numpy(), 2048))
    np.testing.assert_array_equal(f32(actual)[0], logical[17])


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize("rows,n,k", [(1, 2048, 2048), (32, 2048, 2048), (300, 520, 2048), (70, 4096, 512)])
def test_grad_input_of_small_calls_splits_the_reduction(ops, oracle, qname, rows, n, k):
    """Calls of few rows cut the reduction over the weight rows into ranges (16, 16, 4 with uneven ranges, 16) whose
    fp32 partial results a second kernel adds in a fixed order: same bar as the single-pass kernel, a one-hot
    cotangent still returns the weight row exactly, and a repeated call returns the same bits."""
    _, _, synth = ops
    qtype = QTYPES[qname]
    host, device = _weight(synth, qtype, n, k, seed=4321 + qtype)
    grad_output = random_bf16((rows, n), seed=1357)
    actual = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad_output, device, qtype, k)
    assert_matches_f32_reference(actual, oracle.grad_input(qtype, bits(grad_output), host.numpy(), n, k), accumulate_noise=2e-6)
    again = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad_output, device, qtype, k)
    torch.testing.assert_close(again, actual, rtol=0, atol=0)
    one_hot = torch.zeros(rows, n, device="cuda", dtype=torch.bfloat16)
    one_hot[rows - 1, n - 3] = 1
    picked = torch.ops.torch_ggml_ops.mmq_grad_input.default(one_hot, device, qtype, k)
    logical = oracle.bf16_to_f32(oracle.dequant_bf16(qtype, host.numpy(), k))
    np.testing.assert_array_equal(f32(picked)[rows - 1], logical[n - 3])
    assert not f32(picked)[: rows - 1].any()


@pytest.mark.parametrize("qname", ("Q3_K", "Q6_K", "IQ2_S"))
@pytest.mark.parametrize("rows,n,k", [(70, 136, 768), (300, 136, 768), (70, 37, 768), (300, 72, 1280)])
def test_blocks_at_every_even_misalignment(ops, oracle, qname, rows, n, k):
    """Blocks of 110, 210 and 82 bytes start at every even offset inside the 16-byte units the kernels fetch them in.
    With K = 768 or 1280 a weight row is 2 (mod 4) bytes long, so that offset also changes from row to row; 37 rows of
    such a weight do not end on a unit boundary, which selects the 2-byte copy instead.  Forward against the oracle,
    grad-input against the oracle, and a one-hot cotangent returns a weight row bit for bit."""
    tgo, _, synth = ops
    qtype = QTYPES[qname]
    host, device = _weight(synth, qtype, n, k, seed=2468 + qtype)
    x = random_bf16((rows, k), seed=97)
    actual = tgo.mmq(x, device, qtype, n)
    assert_matches_f32_reference(actual, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k))
    grad_output = random_bf16((rows, n), seed=98)
    grad = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad_output, device, qtype, k)
    assert_matches_f32_reference(grad, oracle.grad_input(qtype, bits(grad_output), host.numpy(), n, k), accumulate_noise=2e-6)
    logical = oracle.bf16_to_f32(oracle.dequant_bf16(qtype, host.numpy(), k))
    for column in (0, n // 2 + 1, n - 1):
        one_hot = torch.zeros(rows, n, device="cuda", dtype=torch.bfloat16)
        one_hot[rows - 1, column] = 1
        picked = torch.ops.torch_ggml_ops.mmq_grad_input.default(one_hot, device, qtype, k)
        np.testing.assert_array_equal(f32(picked)[rows - 1], logical[column])


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize("rows,n", [(10, 37), (129, 64), (260, 200)])
def test_grad_input_is_logical_weight_jacobian(ops, oracle, qname, rows, n):
    tgo, _, synth = ops
    qtype, k = QTYPES[qname], 1024
    host, device = _weight(synth, qtype, n, k, seed=5678 + qtype)
    x = random_bf16((rows, k), seed=5678).requires_grad_(True)
    grad_output = random_bf16((rows, n), seed=8765)
    tgo.mmq(x, device, qtype, n).backward(grad_output)
    expected = oracle.grad_input(qtype, bits(grad_output), host.numpy(), n, k)
    # fp32 accumulation of exact bf16 products: only the final rounding separates it from float64
    assert_matches_f32_reference(x.grad, expected, accumulate_noise=2e-6)
    assert device.grad is None


def test_zero_input_and_current_stream(ops):
    tgo, _, synth = ops
    _, device = _weight(synth, 12, 37, 2048, seed=3)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        x = torch.zeros(129, 2048, device="cuda", dtype=torch.bfloat16)
        output = tgo.mmq(x, device, 12, 37)
        grad_output = torch.ones(129, 37, device="cuda", dtype=torch.bfloat16)
        grad_input = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad_output, device, 12, 2048)
        forward_checksum = output.float().abs().sum()
        backward_checksum = grad_input.float().abs().sum()
    stream.synchronize()
    assert forward_checksum.item() == 0.0
    assert backward_checksum.item() > 0.0
    assert torch.isfinite(grad_input).all()


def test_opcheck_and_compile(ops):
    tgo, _, synth = ops
    _, device = _weight(synth, 12, 37, 2048, seed=4)
    x = torch.randn(2, 2048, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    result = torch.library.opcheck(
        torch.ops.torch_ggml_ops.mmq.default,
        (x, device, 12, 37),
        test_utils=("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic"),
        raise_exception=False,
    )
    assert all(value == "SUCCESS" for value in result.values()), result
    grad_output = torch.randn(2, 37, device="cuda", dtype=torch.bfloat16)
    grad_result = torch.library.opcheck(
        torch.ops.torch_ggml_ops.mmq_grad_input.default,
        (grad_output, device, 12, 2048),
        test_utils=("test_schema", "test_faketensor", "test_aot_dispatch_dynamic"),
        raise_exception=False,
    )
    assert all(value == "SUCCESS" for value in grad_result.values()), grad_result

    @torch.compile(fullgraph=True, backend="aot_eager")
    def compiled(x, packed):
        return tgo.mmq(x, packed, 12, 37)

    expected = tgo.mmq(x.detach(), device, 12, 37)
    torch.testing.assert_close(compiled(x.detach(), device), expected, rtol=0, atol=0)


def test_invalid_inputs_fail_without_hidden_copies(ops):
    tgo, _, synth = ops
    _, device = _weight(synth, 12, 37, 2048, seed=5)
    x = torch.randn(4, 2048, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="contiguous"):
        tgo.mmq(x[:, ::2], device, 12, 37)
    with pytest.raises(RuntimeError, match="zero storage offset"):
        tgo.mmq(x[1:], device, 12, 37)
    with pytest.raises(RuntimeError, match="expected"):
        tgo.mmq(x, device.reshape(-1)[:-1].clone(), 12, 37)
    with pytest.raises(RuntimeError, match="unsupported quant_type"):
        tgo.mmq(x, device, 10, 37)
    with pytest.raises(RuntimeError, match="zero-row"):
        tgo.mmq(x[:0], device, 12, 37)

    op = torch.ops.torch_ggml_ops.mmq_grad_input.default
    grad_output = torch.randn(4, 37, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="contiguous"):
        op(grad_output[:, ::2], device, 12, 2048)
    with pytest.raises(RuntimeError, match="zero storage offset"):
        op(grad_output[1:], device, 12, 2048)
    with pytest.raises(RuntimeError, match="expected"):
        op(grad_output, device.reshape(-1)[:-1].clone(), 12, 2048)
    with pytest.raises(RuntimeError, match="unsupported quant_type"):
        op(grad_output, device, 10, 2048)
    with pytest.raises(RuntimeError, match="zero-row"):
        op(grad_output[:0], device, 12, 2048)


def test_grad_input_rejects_higher_order_gradients(ops):
    _, _, synth = ops
    _, device = _weight(synth, 12, 37, 2048, seed=6)
    grad_output = torch.randn(2, 37, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    grad_input = torch.ops.torch_ggml_ops.mmq_grad_input.default(grad_output, device, 12, 2048)
    with pytest.raises(RuntimeError, match="does not support higher-order"):
        grad_input.sum().backward()


def test_c_abi_rejects_bad_arguments_without_launching(ops):
    _, native, _ = ops
    lib = native.lib
    buffer = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = buffer.data_ptr()
    assert lib.tgo_mmq_forward(p, p, p, p, 4, 300, 8, 12, None) == 1
    assert b"multiple of 256" in lib.tgo_last_error()
    assert lib.tgo_mmq_forward(p, p + 2, p, p, 4, 256, 8, 12, None) == 1
    assert b"16-byte aligned" in lib.tgo_last_error()
    assert lib.tgo_mmq_grad_input(p, p, p, p, 4, 8, 256, 99, None) == 1
    assert b"unsupported quant_type" in lib.tgo_last_error()
    assert lib.tgo_dequant_bf16(None, p, 4, 256, 12, None) == 1
    assert lib.tgo_last_error().startswith(b"packed_weight")
