"""The forward kernels under every kind of matrix operand (run with -m gpu).

The library multiplies int8 values, fp16 numbers that hold the same integers exactly, or fp16 numbers that
carry the scales as well (`tgo_set_forward_operand`); by default the format and the size of the call decide.
Every check here runs once with each kind forced, for all five formats: the quantizer's workspace against
the oracle bit for bit, dense, grouped, pair and fused-SwiGLU results against the oracle's forward algebra,
dense == grouped bit for bit, and the kinds against each other (int8 and exact fp16: same integers, different
order of the fp32 scale products; scaled: two fp16 roundings per product on top).
"""

import numpy as np
import pytest
import torch

from helpers import OPERAND_NOISE, QTYPES, assert_matches_f32_reference, bits, f32, max_rel_to_peak, nrmse, random_bf16

pytestmark = pytest.mark.gpu

FORWARD_TOLERANCE = 1e-2   # against dequantize-then-matmul, as in the dense tests


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth
    from torch_ggml_ops import _native

    assert torch.cuda.is_available()
    return torch_ggml_ops, _native, synth


@pytest.fixture(params=("int8", "half", "scaled"))
def operand(request, ops):
    _, native, _ = ops
    native.set_forward_operand(request.param)
    assert native.forward_operand() == request.param
    yield request.param
    native.set_forward_operand("auto")


def _metadata(experts, offsets):
    return (
        torch.tensor(experts, device="cuda", dtype=torch.int64),
        torch.tensor(offsets, device="cuda", dtype=torch.int32),
    )


def test_setting_is_validated_and_defaults_to_auto(ops):
    _, native, _ = ops
    assert native.forward_operand() == "auto"
    assert native.lib.tgo_set_forward_operand(7) != 0
    assert "operand" in native.lib.tgo_last_error().decode()
    assert native.forward_operand() == "auto"


@pytest.mark.parametrize("rows,k", [(33, 512), (129, 2048)])
def test_workspace_holds_the_oracle_quants(ops, oracle, operand, rows, k):
    """The format-less quantizer entry follows a forced exact kind (int8 when the scaled kind is forced); its fp16
    tiles unpack to the same int8 values."""
    _, native, _ = ops
    x = random_bf16((rows, k), seed=70 + rows, scale=2.0)
    x[0, :32] = 0
    x[0, 32:64] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 126.5, -126.5, -0.25, 0.25, -0.0, 3.5, -3.5] * 2)
    workspace = torch.empty(native.lib.tgo_q8_workspace_bytes(rows, k), dtype=torch.uint8, device="cuda")
    native.check(native.lib.tgo_quantize_q8_1(x.data_ptr(), workspace.data_ptr(), rows, k, None))
    q = torch.empty(rows, k, dtype=torch.int8, device="cuda")
    d = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    s = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    native.check(native.lib.tgo_q8_workspace_unpack(workspace.data_ptr(), q.data_ptr(), d.data_ptr(), s.data_ptr(), rows, k, None))
    torch.cuda.synchronize()
    q_ref, d_ref, s_ref = oracle.quantize_q8_1(bits(x))
    np.testing.assert_array_equal(q.cpu().numpy(), q_ref)
    np.testing.assert_array_equal(d.cpu().numpy().view(np.uint32), d_ref.view(np.uint32))
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize("rows,n,k", [(33, 37, 2048), (96, 130, 512), (300, 96, 2048), (129, 264, 768), (640, 128, 256)])
def test_dense_forward_matches_oracle(ops, oracle, operand, qname, rows, n, k):
    """Row counts around the 32- and 128-row tiles, partial column tiles, odd row strides, K of one to eight
    super-blocks (768: blocks of the 2-byte aligned formats at every misalignment)."""
    tgo, _, synth = ops
    qtype = QTYPES[qname]
    host = synth.random_packed_weight(qtype, (n,), k, seed=500 + qtype + n)
    x = random_bf16((rows, k), seed=rows + k)
    actual = tgo.mmq(x, host.cuda(), qtype, n)
    assert torch.isfinite(actual).all()
    assert_matches_f32_reference(actual, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k), OPERAND_NOISE[operand])
    expected = oracle.linear_forward(qtype, bits(x), host.numpy(), n, k)
    assert nrmse(f32(actual), expected) < FORWARD_TOLERANCE
    assert max_rel_to_peak(f32(actual), expected) < FORWARD_TOLERANCE


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_extreme_blocks_stay_exact(ops, oracle, operand, qname):
    """All-ones block bytes (largest quants and sub-scales) against activations of +-amax only: the integer dot
    products reach their largest magnitudes, which the fp16 operands must still hold exactly."""
    tgo, native, _ = ops
    qtype, rows, n, k = QTYPES[qname], 64, 64, 512
    block = native.lib.tgo_block_bytes(qtype)
    rng = np.random.default_rng(qtype)
    raw = np.full((n, k // 256, block), 0xFF, dtype=np.uint8)
    raw[n // 2 :] = rng.choice(np.array([0x00, 0xFF, 0x80, 0x7F], dtype=np.uint8), size=raw[n // 2 :].shape)
    scale_offsets = {11: (108,), 12: (0, 2), 13: (0, 2), 14: (208,), 22: (0,)}[qtype]
    for offset in scale_offsets:   # fp16 super-block scales: 2^-7, so nothing overflows
        raw[:, :, offset] = 0x00
        raw[:, :, offset + 1] = 0x20
    host = torch.from_numpy(raw.reshape(n, -1))
    signs = torch.from_numpy(rng.choice(np.array([-1.0, 1.0], dtype=np.float32), size=(rows, k)))
    x = (signs * 3.0).to(torch.bfloat16).cuda()
    actual = tgo.mmq(x, host.cuda(), qtype, n)
    assert_matches_f32_reference(actual, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k), OPERAND_NOISE[operand])


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_grouped_forward_matches_oracle_and_dense(ops, oracle, operand, qname):
    """Groups of 1 to 300 rows (narrow tasks, partial tiles, a group that spans two tiles of either row tile); every group's slice is
    also bit-identical to the dense operator on that slice."""
    tgo, _, synth = ops
    qtype, n, k = QTYPES[qname], 200, 1024
    host = synth.random_packed_weight(qtype, (6, n), k, seed=600 + qtype)
    device = host.cuda()
    experts, sizes = [5, 0, 2, 3, 1], [1, 33, 300, 31, 97]
    offsets = np.cumsum(sizes).tolist()
    x = random_bf16((offsets[-1], k), seed=4321)
    actual = tgo.grouped_mmq(x, device, *_metadata(experts, offsets), qtype, n)
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    assert_matches_f32_reference(actual, exact, OPERAND_NOISE[operand])
    begin = 0
    for expert, end in zip(experts, offsets):
        if end - begin > 32:   # (up to 32 rows a dense call takes the GEMV family, another summation order)
            dense = tgo.mmq(x[begin:end].clone(), device[expert].clone(), qtype, n)
            torch.testing.assert_close(actual[begin:end], dense, rtol=0, atol=0)
        begin = end


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_pair_and_fused_swiglu(ops, oracle, operand, qname):
    tgo, _, synth = ops
    qtype, n, k = QTYPES[qname], 96, 512
    gate_host = synth.random_packed_weight(qtype, (8, n), k, seed=700 + qtype)
    up_host = synth.random_packed_weight(qtype, (8, n), k, seed=710 + qtype)
    experts, sizes = [0, 2, 5, 7], [5, 140, 64, 33]
    offsets = np.cumsum(sizes).tolist()
    metadata = _metadata(experts, offsets)
    x = random_bf16((offsets[-1], k), seed=88)
    gate, up = tgo.grouped_mmq_pair(x, gate_host.cuda(), up_host.cuda(), *metadata, qtype, n)
    torch.testing.assert_close(gate, tgo.grouped_mmq(x, gate_host.cuda(), *metadata, qtype, n), rtol=0, atol=0)
    torch.testing.assert_close(up, tgo.grouped_mmq(x, up_host.cuda(), *metadata, qtype, n), rtol=0, atol=0)
    gate_ref = oracle.grouped(oracle.mmq_forward, qtype, bits(x), gate_host.numpy(), experts, offsets, n, k, n)
    up_ref = oracle.grouped(oracle.mmq_forward, qtype, bits(x), up_host.numpy(), experts, offsets, n, k, n)
    assert_matches_f32_reference(gate, gate_ref, OPERAND_NOISE[operand])
    assert_matches_f32_reference(up, up_ref, OPERAND_NOISE[operand])
    activated = tgo.grouped_mmq_swiglu(x, gate_host.cuda(), up_host.cuda(), *metadata, qtype, n)
    gate_bf16 = torch.from_numpy(gate_ref).to(torch.bfloat16).double().numpy()
    with np.errstate(over="ignore"):
        expected = gate_bf16 / (1.0 + np.exp(-gate_bf16)) * up_ref.astype(np.float64)
    assert nrmse(f32(activated), expected) < 5e-3
    # (the scaled kind's operand rounding reaches both factors of the product)
    assert max_rel_to_peak(f32(activated), expected) < (1.5e-2 if operand == "scaled" else 1e-2)


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_kinds_agree(ops, qname):
    """int8 against exact fp16: same integer dot products, fp32 scale products in a different order, so the results
    differ by fp32 rounding before the final bf16 rounding, i.e. at most one bf16 ulp here and there.  The scaled
    kind adds two fp16 roundings per product.  A small call under "auto" takes the exact kind of its format."""
    tgo, native, synth = ops
    qtype, rows, n, k = QTYPES[qname], 300, 256, 2048
    weight = synth.random_packed_weight(qtype, (n,), k, seed=800 + qtype).cuda()
    x = random_bf16((rows, k), seed=55)
    results = {}
    try:
        for kind in ("int8", "half", "scaled"):
            native.set_forward_operand(kind)
            results[kind] = f32(tgo.mmq(x, weight, qtype, n)).astype(np.float64)
    finally:
        native.set_forward_operand("auto")
    peak = np.abs(results["int8"]).max()
    difference = np.abs(results["int8"] - results["half"])
    assert (difference <= np.abs(results["int8"]) * 2.0**-7 + 1e-6 * peak).all()
    assert nrmse(results["half"], results["int8"]) < 1e-3
    difference = np.abs(results["int8"] - results["scaled"])
    assert (difference <= np.abs(results["int8"]) * 2.0**-7 + OPERAND_NOISE["scaled"] * peak).all()
    assert nrmse(results["scaled"], results["int8"]) < 2e-3
    assert native.forward_operand_for(qtype, rows, n) == ("half" if qname == "IQ2_S" else "int8")
    chosen = f32(tgo.mmq(x, weight, qtype, n)).astype(np.float64)
    np.testing.assert_array_equal(chosen, results["half" if qname == "IQ2_S" else "int8"])


@pytest.mark.parametrize("qname", ("IQ2_S", "Q5_K"))
@pytest.mark.parametrize("rows,n", [(300, 256), (2048, 2048)])
def test_workspace_of_a_forward_call_unpacks_by_its_tag(ops, oracle, qname, rows, n):
    """Under "auto" the kind depends on the call (here: exact fp16 or int8 for the small one, scaled for the large
    one), so whoever reads the workspace afterwards cannot derive its layout from the setting: the unpacker follows
    the tag that the quantizer left in the workspace.  All layouts give back the oracle's quants, scales and sums."""
    _, native, synth = ops
    qtype, k = QTYPES[qname], 512
    assert native.forward_operand() == "auto"
    assert native.forward_operand_for(qtype, rows, n) == ("scaled" if rows == 2048 else "half" if qname == "IQ2_S" else "int8")
    weight = synth.random_packed_weight(qtype, (n,), k, seed=900 + qtype).cuda()
    x = random_bf16((rows, k), seed=91, scale=2.0)
    out = torch.empty(rows, n, dtype=torch.bfloat16, device="cuda")
    workspace = torch.empty(native.lib.tgo_q8_workspace_bytes(rows, k), dtype=torch.uint8, device="cuda")
    native.check(native.lib.tgo_mmq_forward(x.data_ptr(), weight.data_ptr(), out.data_ptr(), workspace.data_ptr(), rows, k, n, qtype, None))
    q = torch.empty(rows, k, dtype=torch.int8, device="cuda")
    d = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    s = torch.empty(rows, k // 32, dtype=torch.float32, device="cuda")
    native.check(native.lib.tgo_q8_workspace_unpack(workspace.data_ptr(), q.data_ptr(), d.data_ptr(), s.data_ptr(), rows, k, None))
    torch.cuda.synchronize()
    q_ref, d_ref, s_ref = oracle.quantize_q8_1(bits(x))
    np.testing.assert_array_equal(q.cpu().numpy(), q_ref)
    np.testing.assert_array_equal(d.cpu().numpy().view(np.uint32), d_ref.view(np.uint32))
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))


def test_prepared_forward_refuses_a_workspace_of_another_kind(ops):
    """A workspace quantized under one forced kind and multiplied under another: every output is NaN."""
    tgo, native, synth = ops
    qtype, rows, n, k = QTYPES["Q4_K"], 64, 64, 512
    weight = synth.random_packed_weight(qtype, (n,), k, seed=77).cuda()
    x = random_bf16((rows, k), seed=3)
    workspace = torch.empty(native.lib.tgo_q8_workspace_bytes(rows, k), dtype=torch.uint8, device="cuda")
    out = torch.zeros(rows, n, dtype=torch.bfloat16, device="cuda")
    try:
        native.set_forward_operand("half")
        native.check(native.lib.tgo_quantize_q8_1(x.data_ptr(), workspace.data_ptr(), rows, k, None))
        native.check(native.lib.tgo_mmq_forward_prepared(workspace.data_ptr(), weight.data_ptr(), out.data_ptr(), rows, k, n, qtype, None))
        torch.cuda.synchronize()
        assert torch.isfinite(out).all()
        torch.testing.assert_close(out, tgo.mmq(x, weight, qtype, n), rtol=0, atol=0)
        native.set_forward_operand("int8")
        native.check(native.lib.tgo_mmq_forward_prepared(workspace.data_ptr(), weight.data_ptr(), out.data_ptr(), rows, k, n, qtype, None))
        torch.cuda.synchronize()
        assert torch.isnan(out).all()
    finally:
        native.set_forward_operand("auto")


@pytest.mark.parametrize("seed", range(10))
def test_ragged_groups_of_any_mix_under_the_scaled_kind(ops, oracle, seed):
    """Seeded random group lists for the two kernels of the scaled kind: empty groups, whole groups of at most 32 rows
    (their own kernel, listed behind the others), groups that end a few rows into a 256-row tile, repeated and
    unsorted experts, column counts off the 128-column tile and off the 16-byte stores, one or two projections."""
    tgo, native, synth = ops
    rng = np.random.default_rng(9000 + seed)
    qtype = list(QTYPES.values())[seed % len(QTYPES)]
    n = int(rng.choice([37, 128, 200, 264]))
    k = int(rng.choice([256, 768, 1024]))
    experts_total = 16
    groups = int(rng.integers(5, 14))
    sizes = rng.choice([0, 1, 2, 31, 32, 33, 64, 255, 256, 257, 300, 520], size=groups).tolist()
    if sum(sizes) == 0:
        sizes[0] = 40
    experts = rng.integers(0, experts_total, size=groups).tolist()
    offsets = np.cumsum(sizes).tolist()
    first_host = synth.random_packed_weight(qtype, (experts_total, n), k, seed=100 + seed)
    second_host = synth.random_packed_weight(qtype, (experts_total, n), k, seed=200 + seed)
    x = random_bf16((offsets[-1], k), seed=300 + seed)
    metadata = _metadata(experts, offsets)
    native.set_forward_operand("scaled")
    try:
        if seed % 2 == 0:
            first, second = tgo.grouped_mmq_pair(x, first_host.cuda(), second_host.cuda(), *metadata, qtype, n)
        else:
            first, second = tgo.grouped_mmq(x, first_host.cuda(), *metadata, qtype, n), None
    finally:
        native.set_forward_operand("auto")
    expected = oracle.grouped(oracle.mmq_forward, qtype, bits(x), first_host.numpy(), experts, offsets, n, k, n)
    assert_matches_f32_reference(first, expected, OPERAND_NOISE["scaled"])
    if second is not None:
        expected = oracle.grouped(oracle.mmq_forward, qtype, bits(x), second_host.numpy(), experts, offsets, n, k, n)
        assert_matches_f32_reference(second, expected, OPERAND_NOISE["scaled"])


@pytest.mark.parametrize("grouped", (False, True))
def test_more_tiles_than_one_table_per_cu_holds(ops, grouped):
    """16 384 rows x 32 896 outputs: 64 row tasks x 257 column tiles, more than the 64 items that each of the 256
    workgroups of the scaled kernel keeps in its table, so the launch grows its grid.  Checked against the int8 kind
    (itself pinned on the oracle at the sizes the oracle finishes)."""
    tgo, native, synth = ops
    qtype, rows, n, k = QTYPES["Q4_K"], 16384, 32896, 256
    weight = synth.random_packed_weight(qtype, (4, n) if grouped else (n,), k, seed=77).cuda()
    x = random_bf16((rows, k), seed=78)
    metadata = _metadata([1, 3, 0], [5000, 5020, rows])

    def run():
        return tgo.grouped_mmq(x, weight, *metadata, qtype, n) if grouped else tgo.mmq(x, weight, qtype, n)

    assert native.forward_operand_for(qtype, rows, n) == "scaled"
    scaled = run()
    native.set_forward_operand("int8")
    try:
        exact = run()
    finally:
        native.set_forward_operand("auto")
    peak = float(exact.float().abs().max())
    step = 1 << 22   # (compared in slices: the fp32 copies of a gigabyte of bf16 would be four)
    flat_scaled, flat_exact = scaled.view(-1), exact.view(-1)
    for begin in range(0, flat_exact.numel(), step * 16):
        a = flat_scaled[begin : begin + step * 16].float()
        b = flat_exact[begin : begin + step * 16].float()
        assert bool(((a - b).abs() <= b.abs() * 2.0**-7 + OPERAND_NOISE["scaled"] * peak).all())


@pytest.mark.parametrize("k", (512, 1024))
@pytest.mark.parametrize("sizes", ([1, 5, 32, 17, 31, 2], [40, 300, 33], [7, 0, 290, 32, 0, 64]))
def test_only_short_groups_only_long_groups_and_both(ops, oracle, k, sizes):
    """The scaled kind serves groups of at most 32 rows and the others with different workgroups (of one launch for rows
    of four super-blocks or more, k = 1024; of two launches below that, k = 512): lists that have only the one kind, only
    the other, and both with empty groups in between."""
    tgo, native, synth = ops
    qtype, n = QTYPES["Q4_K"], 200
    experts = list(range(len(sizes)))[::-1]
    offsets = np.cumsum(sizes).tolist()
    host = synth.random_packed_weight(qtype, (len(sizes), n), k, seed=400 + k)
    x = random_bf16((offsets[-1], k), seed=401)
    native.set_forward_operand("scaled")
    try:
        actual = tgo.grouped_mmq(x, host.cuda(), *_metadata(experts, offsets), qtype, n)
    finally:
        native.set_forward_operand("auto")
    expected = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), experts, offsets, n, k, n)
    assert_matches_f32_reference(actual, expected, OPERAND_NOISE["scaled"])
