"""GPU parity of the grouped and fused-pair operators against the CPU oracle (-m gpu).

Mirrors the reference's tests/test_grouped_mmq.py: the same group layouts
([1,128,257,262] with experts [0,2,5,7]; [65,194,323,512]; [2,5,6]; the boundary sizes
1,15,16,17,63,64,65,127,128,129), synthetic seeded blocks in place of its checkpoint.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits, f32, forward_noise, max_rel_to_peak, nrmse, random_bf16

pytestmark = pytest.mark.gpu

FORWARD_TOLERANCE = 1e-2
BOUNDARY_SIZES = (1, 15, 16, 17, 63, 64, 65, 127, 128, 129)


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


def _experts(synth, qtype, experts, n, k, seed):
    host = synth.random_packed_weight(qtype, (experts, n), k, seed=seed)
    return host, host.cuda()


def _metadata(experts, offsets):
    return (
        torch.tensor(experts, device="cuda", dtype=torch.int64),
        torch.tensor(offsets, device="cuda", dtype=torch.int32),
    )


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_grouped_forward_matches_oracle(ops, oracle, qname):
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 37, 2048
    host, device = _experts(synth, qtype, 8, n, k, seed=10 + qtype)
    experts, offsets = [0, 2, 5, 7], [1, 128, 257, 262]
    x = random_bf16((262, k), seed=3456)
    actual = tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n)
    assert actual.shape == (262, n) and actual.dtype == torch.bfloat16 and actual.is_contiguous()
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    assert_matches_f32_reference(actual, exact)
    logical = oracle.grouped(oracle.linear_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    assert nrmse(f32(actual), logical) < FORWARD_TOLERANCE
    assert max_rel_to_peak(f32(actual), logical) < FORWARD_TOLERANCE


@pytest.mark.parametrize("qname", ("Q4_K", "IQ2_S"))
def test_grouped_forward_equals_dense_per_expert(ops, qname):
    """Each group's slice is bit-identical to the dense operator on that slice."""
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 512, 2048
    _, device = _experts(synth, qtype, 6, n, k, seed=20 + qtype)
    experts, offsets = [0, 1, 3, 4], [65, 194, 323, 512]
    x = random_bf16((512, k), seed=2468)
    grouped = tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n)
    begin = 0
    for expert, end in zip(experts, offsets):
        dense = tgo.mmq(x[begin:end].clone(), device[expert].clone(), qtype, n)
        torch.testing.assert_close(grouped[begin:end], dense, rtol=0, atol=0)
        begin = end


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_pair_forward_equals_two_single_calls(ops, qname):
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 37, 2048
    _, first = _experts(synth, qtype, 8, n, k, seed=30 + qtype)
    _, second = _experts(synth, qtype, 8, n, k, seed=40 + qtype)
    metadata = _metadata([0, 2, 5, 7], [1, 128, 257, 262])
    x = random_bf16((262, k), seed=9012)
    out_first, out_second = tgo.grouped_mmq_pair(x, first, second, *metadata, qtype, n)
    torch.testing.assert_close(out_first, tgo.grouped_mmq(x, first, *metadata, qtype, n), rtol=0, atol=0)
    torch.testing.assert_close(out_second, tgo.grouped_mmq(x, second, *metadata, qtype, n), rtol=0, atol=0)


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_grouped_grad_input_matches_oracle(ops, oracle, qname):
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 37, 512
    host, device = _experts(synth, qtype, 4, n, k, seed=50 + qtype)
    experts, offsets = [0, 1, 3], [2, 5, 6]
    x = random_bf16((6, k), seed=8642).requires_grad_(True)
    grad_output = random_bf16((6, n), seed=2486)
    tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n).backward(grad_output)
    expected = oracle.grouped(oracle.grad_input, qtype, bits(grad_output), host.numpy(), experts, offsets, n, k, k)
    assert_matches_f32_reference(x.grad, expected, accumulate_noise=2e-6)


@pytest.mark.parametrize("qname", ("Q4_K", "Q6_K", "IQ2_S"))
def test_grouped_grad_input_group_boundaries(ops, oracle, qname):
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 64, 512
    host, device = _experts(synth, qtype, len(BOUNDARY_SIZES), n, k, seed=60 + qtype)
    offsets = np.cumsum(BOUNDARY_SIZES).tolist()
    experts = list(range(len(BOUNDARY_SIZES)))[::-1]
    rows = offsets[-1]
    grad_output = random_bf16((rows, n), seed=1357)
    actual = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(
        grad_output, device, *_metadata(experts, offsets), qtype, k
    )
    expected = oracle.grouped(oracle.grad_input, qtype, bits(grad_output), host.numpy(), experts, offsets, n, k, k)
    assert_matches_f32_reference(actual, expected, accumulate_noise=2e-6)


@pytest.mark.parametrize("qname", ("Q3_K", "Q5_K"))
def test_grouped_forward_group_boundaries(ops, oracle, qname):
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 96, 512
    host, device = _experts(synth, qtype, len(BOUNDARY_SIZES), n, k, seed=70 + qtype)
    offsets = np.cumsum(BOUNDARY_SIZES).tolist()
    experts = list(range(len(BOUNDARY_SIZES)))
    x = random_bf16((offsets[-1], k), seed=7531)
    actual = tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n)
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    assert_matches_f32_reference(actual, exact)
    logical = oracle.grouped(oracle.linear_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    assert nrmse(f32(actual), logical) < FORWARD_TOLERANCE
    assert max_rel_to_peak(f32(actual), logical) < FORWARD_TOLERANCE


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_pair_grad_input_sums_both_projections_once(ops, oracle, qname):
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 37, 512
    host_first, first = _experts(synth, qtype, 8, n, k, seed=80 + qtype)
    host_second, second = _experts(synth, qtype, 8, n, k, seed=90 + qtype)
    experts, offsets = [0, 2, 5, 7], [1, 128, 257, 262]
    x = random_bf16((262, k), seed=1111).requires_grad_(True)
    grad_first = random_bf16((262, n), seed=2222)
    grad_second = random_bf16((262, n), seed=3333)
    out_first, out_second = tgo.grouped_mmq_pair(x, first, second, *_metadata(experts, offsets), qtype, n)
    torch.autograd.backward((out_first, out_second), (grad_first, grad_second))
    expected = oracle.grouped(oracle.grad_input, qtype, bits(grad_first), host_first.numpy(), experts, offsets, n, k, k)
    expected = expected.astype(np.float64) + oracle.grouped(
        oracle.grad_input, qtype, bits(grad_second), host_second.numpy(), experts, offsets, n, k, k
    )
    assert_matches_f32_reference(x.grad, expected.astype(np.float32), accumulate_noise=2e-6)

    # only one cotangent defined: falls back to the single-projection operator
    y = random_bf16((262, k), seed=1111).requires_grad_(True)
    only_first, _ = tgo.grouped_mmq_pair(y, first, second, *_metadata(experts, offsets), qtype, n)
    only_first.backward(grad_first)
    single = oracle.grouped(oracle.grad_input, qtype, bits(grad_first), host_first.numpy(), experts, offsets, n, k, k)
    assert_matches_f32_reference(y.grad, single, accumulate_noise=2e-6)


@pytest.mark.parametrize("qname", ("Q4_K", "Q5_K"))
def test_pair_grad_input_many_tasks_per_workgroup(ops, oracle, qname):
    """More (task, column tile) items than CUs: every workgroup of the persistent grad-input kernel walks
    several items back to back, with groups that span row tiles, empty groups, single rows and an
    out_features (100) that is not a multiple of the 64-row reduction step."""
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 100, 2048
    sizes = [300, 1, 257, 0, 64, 513, 31, 2, 128, 129, 7, 256, 0, 65, 90, 33, 1, 255, 17, 40, 3, 100, 64, 5, 260, 12, 1, 77, 48, 9]
    experts = [(7 * i + 3) % 32 for i in range(len(sizes))]
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    host_first, first = _experts(synth, qtype, 32, n, k, seed=180 + qtype)
    host_second, second = _experts(synth, qtype, 32, n, k, seed=190 + qtype)
    grad_first = random_bf16((rows, n), seed=4444)
    grad_second = random_bf16((rows, n), seed=5555)
    actual = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
        grad_first, grad_second, first, second, *_metadata(experts, offsets), qtype, k
    )
    expected = oracle.grouped(oracle.grad_input, qtype, bits(grad_first), host_first.numpy(), experts, offsets, n, k, k)
    expected = expected.astype(np.float64) + oracle.grouped(
        oracle.grad_input, qtype, bits(grad_second), host_second.numpy(), experts, offsets, n, k, k
    )
    assert_matches_f32_reference(actual, expected.astype(np.float32), accumulate_noise=2e-6)


@pytest.mark.parametrize("sources", (1, 2))
@pytest.mark.parametrize("n", (64, 128, 192, 200, 296, 512))
@pytest.mark.parametrize("qname", ("Q4_K", "Q5_K"))
def test_role_split_kernel_every_prefetch_phase(ops, oracle, qname, n, sources):
    """The persistent grad-input kernel of Q4_K / Q5_K keeps the packed blocks of four reduction steps and the
    cotangent fragments of two in flight in rings of registers.  With 1, 2, 3, 4 (200 columns: uneven last step),
    5 and 8 steps per source, one or two sources and several items per workgroup, every ring phase meets every
    position in an item; a one-hot cotangent per step must return that step's weight row exactly (bit for bit),
    and random cotangents must match the oracle.  Groups of 70..300 rows keep the tasks out of the short-task kernel."""
    _check_one_hot_and_random_cotangents(ops, oracle, qname, n, sources, [70, 300, 129], [2, 0, 3])


@pytest.mark.parametrize("sources", (1, 2))
@pytest.mark.parametrize("n", (64, 200, 512))
@pytest.mark.parametrize("qname", ("Q4_K", "Q5_K"))
def test_short_remainders_next_to_full_tiles(ops, oracle, qname, n, sources):
    """Remainders of 1, 18, 32 and 33 rows behind full 256-row tiles (groups of 257, 530, 288 and 289 rows), a group
    of exactly 256 rows and one of 31: the full tiles run in the persistent kernel, the remainders in the short-task
    kernel, and both write neighbouring rows of one output.  Every row gets a one-hot cotangent that must return a
    weight row bit for bit, and random cotangents must match the oracle."""
    _check_one_hot_and_random_cotangents(ops, oracle, qname, n, sources, [257, 31, 288, 256, 289, 530], [1, 3, 0, 2, 5, 4])


def _check_one_hot_and_random_cotangents(ops, oracle, qname, n, sources, sizes, experts):
    tgo, synth = ops
    qtype, k = QTYPES[qname], 1024
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    host = [synth.random_packed_weight(qtype, (max(experts) + 1, n), k, seed=700 + 10 * s + qtype) for s in range(sources)]
    device = [h.cuda() for h in host]
    metadata = _metadata(experts, offsets)
    op_single = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default
    op_pair = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default

    def run(grads):
        if sources == 1:
            return op_single(grads[0], device[0], *metadata, qtype, k)
        return op_pair(grads[0], grads[1], device[0], device[1], *metadata, qtype, k)

    logical = [oracle.bf16_to_f32(oracle.dequant_bf16(qtype, h.numpy(), k)) for h in host]   # [experts, n, k]
    steps = (n + 63) // 64
    # row r of group g gets a one in column (64 * (r % steps) + r % 64) capped at n - 1 of source r % sources
    one_hot = [torch.zeros(rows, n, dtype=torch.bfloat16) for _ in range(sources)]
    picks, begin = [], 0
    for expert, end in zip(experts, offsets):
        for row in range(begin, end):
            column = min(64 * (row % steps) + row % 64, n - 1)
            one_hot[row % sources][row, column] = 1
            picks.append((row, expert, row % sources, column))
        begin = end
    result = f32(run([g.cuda() for g in one_hot]))
    for row, expert, source, column in picks:
        np.testing.assert_array_equal(result[row], logical[source][expert, column], err_msg=f"row {row} column {column}")

    grads = [random_bf16((rows, n), seed=900 + s) for s in range(sources)]
    expected = np.zeros((rows, k), dtype=np.float64)
    for s in range(sources):
        expected += oracle.grouped(oracle.grad_input, qtype, bits(grads[s]), host[s].numpy(), experts, offsets, n, k, k)
    assert_matches_f32_reference(run(grads), expected.astype(np.float32), accumulate_noise=2e-6)


@pytest.mark.parametrize("qname", ("Q4_K", "Q6_K"))
def test_more_groups_than_one_listing_pass(ops, oracle, qname):
    """700 groups: the tile-task list is written 256 groups at a time, and the forward lists tasks of at most
    32 rows behind all the others.  Sizes mix empty groups, short remainders (1..32 rows), remainders just over
    the limit and groups of several row tiles (128-row tiles for Q4_K, 256-row ones for Q6_K)."""
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 24, 256
    palette = (0, 1, 5, 31, 32, 33, 2, 0, 17, 130, 8, 160, 3, 289, 64, 1)
    sizes = [palette[(5 * i + i // 16) % len(palette)] for i in range(700)]
    sizes[300] = 2 * 256 + 32
    sizes[699] = 128 + 32
    experts = [(11 * i + 2) % 700 for i in range(len(sizes))]  # as many experts as groups: the operator's own limit
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    assert rows > 4 * len(sizes)  # the MFMA kernel family, not the decode one
    host, device = _experts(synth, qtype, 700, n, k, seed=380 + qtype)
    x = random_bf16((rows, k), seed=1212)
    actual = tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n)
    assert_matches_f32_reference(actual, oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n),
                                 forward_noise(qtype, x.shape[0], n))
    grad = random_bf16((rows, n), seed=1313)
    actual = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad, device, *_metadata(experts, offsets), qtype, k)
    expected = oracle.grouped(oracle.grad_input, qtype, bits(grad), host.numpy(), experts, offsets, n, k, k)
    assert_matches_f32_reference(actual, expected, accumulate_noise=2e-6)


TASK_LAYOUTS = {
    "seven_tasks": [33] * 7,                                   # fewer tasks than XCDs
    "eight_tasks": [33] * 8,
    "nine_tasks": [33] * 9,
    "only_short": [5, 1, 32, 17, 9, 30, 2, 31, 8, 4, 3, 12, 21],       # every group is listed as a short one
    "only_full": [128] * 19,
    "short_behind_long": [1] * 21 + [300, 260, 140],
    "remainders": [160, 7, 129, 33, 290, 64, 65, 1, 640, 31, 96, 257, 2, 384, 32, 97, 45],
}


@pytest.mark.parametrize("layout", tuple(TASK_LAYOUTS))
@pytest.mark.parametrize("qname", ("Q5_K", "Q3_K"))
def test_every_task_runs_once_whatever_the_list_looks_like(ops, qname, layout):
    """Workgroups find their task through the XCD they run on: each XCD takes a contiguous share of the ordinary
    tasks and one of the short ones.  Whatever the numbers of either kind, the joint call must give every group
    exactly what a call with that group alone gives (same kernels, one task list of its own): a task left out
    leaves rows unwritten, a wrong one writes other values."""
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 128, 512
    sizes = TASK_LAYOUTS[layout]
    experts = [(3 * i + 1) % len(sizes) for i in range(len(sizes))]
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    _, first = _experts(synth, qtype, len(sizes), n, k, seed=410 + qtype)
    _, second = _experts(synth, qtype, len(sizes), n, k, seed=420 + qtype)
    x = random_bf16((rows, k), seed=99)
    grad_first = random_bf16((rows, n), seed=98)
    grad_second = random_bf16((rows, n), seed=97)
    metadata = _metadata(experts, offsets)
    out_first, out_second = tgo.grouped_mmq_pair(x, first, second, *metadata, qtype, n)
    dx = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(grad_first, grad_second, first, second, *metadata, qtype, k)
    dx_single = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad_first, first, *metadata, qtype, k)
    begin = 0
    for expert, end in zip(experts, offsets):
        # (a dense-sized call would take the decode kernels: keep the one-group calls above 4 rows per group)
        if end - begin > 4:
            alone = _metadata([expert], [end - begin])
            one_first, one_second = tgo.grouped_mmq_pair(x[begin:end].clone(), first, second, *alone, qtype, n)
            torch.testing.assert_close(out_first[begin:end], one_first, rtol=0, atol=0)
            torch.testing.assert_close(out_second[begin:end], one_second, rtol=0, atol=0)
            one_dx = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
                grad_first[begin:end].clone(), grad_second[begin:end].clone(), first, second, *alone, qtype, k)
            assert torch.equal(dx[begin:end].view(torch.int16), one_dx.view(torch.int16))
            one_dx = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad_first[begin:end].clone(), first, *alone, qtype, k)
            assert torch.equal(dx_single[begin:end].view(torch.int16), one_dx.view(torch.int16))
        begin = end
    assert torch.isfinite(out_first).all() and torch.isfinite(out_second).all() and torch.isfinite(dx).all()


@pytest.mark.parametrize("qname", ("Q5_K",))
def test_pair_at_benchmark_shape_per_expert(ops, oracle, qname):
    """The benchmark's per-expert shape (out_features 512, in_features 2048: eight reduction steps per source,
    four forward column tiles) with groups from 1 to 300 rows, forward pair and fused grad-input."""
    tgo, synth = ops
    qtype, n, k = QTYPES[qname], 512, 2048
    sizes = [300, 7, 33, 1, 128, 64, 31, 32]
    experts = [5, 0, 3, 7, 1, 6, 2, 4]
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    host_first, first = _experts(synth, qtype, 8, n, k, seed=280 + qtype)
    host_second, second = _experts(synth, qtype, 8, n, k, seed=290 + qtype)
    x = random_bf16((rows, k), seed=6666)
    out_first, out_second = tgo.grouped_mmq_pair(x, first, second, *_metadata(experts, offsets), qtype, n)
    for out, host in ((out_first, host_first), (out_second, host_second)):
        exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
        assert_matches_f32_reference(out, exact)
    grad_first = random_bf16((rows, n), seed=7777)
    grad_second = random_bf16((rows, n), seed=8888)
    actual = torch.ops.torch_ggml_ops.grouped_mmq_pair_grad_input.default(
        grad_first, grad_second, first, second, *_metadata(experts, offsets), qtype, k
    )
    expected = oracle.grouped(oracle.grad_input, qtype, bits(grad_first), host_first.numpy(), experts, offsets, n, k, k)
    expected = expected.astype(np.float64) + oracle.grouped(
        oracle.grad_input, qtype, bits(grad_second), host_second.numpy(), experts, offsets, n, k, k
    )
    assert_matches_f32_reference(actual, expected.astype(np.float32), accumulate_noise=2e-6)


def test_invalid_groups_are_skipped_and_other_rows_untouched(ops, oracle):
    tgo, synth = ops
    qtype, n, k = 12, 64, 256
    host, device = _experts(synth, qtype, 4, n, k, seed=5)
    x = random_bf16((40, k), seed=5)
    # group 1 names an expert that does not exist, group 2 is empty
    experts, offsets = [1, 9, 2, 3], [10, 20, 20, 40]
    actual = tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n)
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    covered = ~np.isnan(exact[:, 0])
    assert covered.sum() == 30
    assert_matches_f32_reference(actual[torch.from_numpy(covered).cuda()], exact[covered])


def test_zero_input_and_current_stream(ops):
    tgo, synth = ops
    _, device = _experts(synth, 12, 8, 37, 2048, seed=6)
    metadata = _metadata([0, 2, 5, 7], [1, 128, 257, 262])
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        x = torch.zeros(262, 2048, device="cuda", dtype=torch.bfloat16)
        first, second = tgo.grouped_mmq_pair(x, device, device, *metadata, 12, 37)
        checksum = first.float().abs().sum() + second.float().abs().sum()
        grad_output = torch.ones(262, 37, device="cuda", dtype=torch.bfloat16)
        grad_input = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad_output, device, *metadata, 12, 2048)
        backward_checksum = grad_input.float().abs().sum()
    stream.synchronize()
    assert checksum.item() == 0.0
    assert backward_checksum.item() > 0.0


def test_opcheck_and_compile(ops):
    tgo, synth = ops
    _, device = _experts(synth, 12, 8, 37, 2048, seed=7)
    metadata = _metadata([0, 2, 5, 7], [1, 128, 257, 262])
    x = torch.randn(262, 2048, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    for op, args in (
        (torch.ops.torch_ggml_ops.grouped_mmq.default, (x, device, *metadata, 12, 37)),
        (torch.ops.torch_ggml_ops.grouped_mmq_pair.default, (x, device, device, *metadata, 12, 37)),
    ):
        result = torch.library.opcheck(
            op,
            args,
            test_utils=("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic"),
            raise_exception=False,
        )
        assert all(value == "SUCCESS" for value in result.values()), result

    @torch.compile(fullgraph=True, backend="aot_eager")
    def compiled(x, packed, experts, offsets):
        return tgo.grouped_mmq(x, packed, experts, offsets, 12, 37)

    expected = tgo.grouped_mmq(x.detach(), device, *metadata, 12, 37)
    torch.testing.assert_close(compiled(x.detach(), device, *metadata), expected, rtol=0, atol=0)


def test_invalid_inputs_fail_without_hidden_copies(ops):
    tgo, synth = ops
    _, device = _experts(synth, 12, 8, 37, 2048, seed=8)
    experts, offsets = _metadata([0, 2, 5, 7], [1, 128, 257, 262])
    x = torch.randn(262, 2048, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="contiguous"):
        tgo.grouped_mmq(x[:, ::2], device, experts, offsets, 12, 37)
    with pytest.raises(RuntimeError, match="zero storage offset"):
        tgo.grouped_mmq(x[1:], device, experts, offsets, 12, 37)
    with pytest.raises(RuntimeError, match="bytes per row"):
        tgo.grouped_mmq(x, device[:, :, :-1].contiguous(), experts, offsets, 12, 37)
    with pytest.raises(RuntimeError, match="unsupported quant_type"):
        tgo.grouped_mmq(x, device, experts, offsets, 10, 37)
    with pytest.raises(RuntimeError, match="zero-row"):
        tgo.grouped_mmq(x[:0], device, experts, offsets, 12, 37)
    with pytest.raises(RuntimeError, match="torch.int32"):
        tgo.grouped_mmq(x, device, experts, offsets.to(torch.int64), 12, 37)
    with pytest.raises(RuntimeError, match="torch.int64"):
        tgo.grouped_mmq(x, device, experts.to(torch.int32), offsets, 12, 37)
    grad_output = torch.randn(262, 37, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    grad_input = torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(grad_output, device, experts, offsets, 12, 2048)
    with pytest.raises(RuntimeError, match="does not support higher-order"):
        grad_input.sum().backward()
