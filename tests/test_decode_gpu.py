"""GPU parity of the decode-regime (GEMV) forward path against the CPU oracle (-m gpu).

Dense calls with at most 8 rows and grouped calls that average at most 4 rows per group
take the bandwidth-oriented kernel; the shapes here cover its edges: 1..8 rows, output
widths that are not a multiple of its 16-row weight tile, K below and above its
2048-value pass, groups of 1..9 rows (more than one task per group) and invalid groups.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits, f32, nrmse, random_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth
    from torch_ggml_ops import _native

    assert torch.cuda.is_available()
    return torch_ggml_ops, _native, synth


def test_kernel_family_selection(ops):
    _, native, _ = ops
    family = native.lib.tgo_forward_kernel_family
    assert family(1, 0) == b"gemv" and family(8, 0) == b"gemv" and family(32, 0) == b"gemv" and family(33, 0) == b"mfma"
    assert family(64, 57) == b"gemv" and family(32768, 256) == b"mfma"


@pytest.mark.parametrize("qname", tuple(QTYPES))
@pytest.mark.parametrize(
    "rows,n,k",
    [(1, 4096, 2048), (2, 48, 768), (3, 37, 512), (4, 33, 1024), (8, 100, 2304), (5, 16, 4352),
     # short K with out_features a multiple of 4 or 2: several weight rows share a pass
     (1, 64, 256), (3, 40, 512), (7, 100, 512), (8, 36, 1024), (2, 20, 512), (1, 2048, 512), (6, 6, 1024),
     # dense calls of 9 to 32 rows are walked eight rows at a time
     (9, 37, 512), (16, 2048, 2048), (17, 48, 768), (26, 100, 2304), (32, 64, 1024)],
)
def test_dense_decode_matches_oracle(ops, oracle, qname, rows, n, k):
    tgo, _, synth = ops
    qtype = QTYPES[qname]
    host = synth.random_packed_weight(qtype, (n,), k, seed=300 + qtype + rows)
    x = random_bf16((rows, k), seed=17 + rows)
    actual = tgo.mmq(x, host.cuda(), qtype, n)
    assert actual.shape == (rows, n) and torch.isfinite(actual).all()
    assert_matches_f32_reference(actual, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k))
    if rows * n >= 512:
        assert nrmse(f32(actual), oracle.linear_forward(qtype, bits(x), host.numpy(), n, k)) < 1e-2


def _shape_sweep():
    """A deterministic spread of small dense shapes: every row count routine (1, 2, 4, 8, matrix-core, walked),
    K of 1..9 super-blocks (long rows of 4, 2 and 1 weight rows, partial last passes), out_features that are and
    are not multiples of 2, 4 and 16."""
    rng = np.random.default_rng(20240607)
    rows = (1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 24, 31, 32)
    outs = (1, 2, 4, 6, 15, 16, 17, 20, 36, 50, 100)
    ks = (256, 512, 768, 1024, 1280, 2048, 2304)
    return sorted({(int(rng.choice(rows)), int(rng.choice(outs)), int(rng.choice(ks))) for _ in range(60)})


@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_dense_decode_shape_sweep(ops, oracle, qname):
    tgo, _, synth = ops
    qtype = QTYPES[qname]
    for rows, n, k in _shape_sweep():
        host = synth.random_packed_weight(qtype, (n,), k, seed=rows * 1000 + n + k)
        x = random_bf16((rows, k), seed=rows + n)
        actual = tgo.mmq(x, host.cuda(), qtype, n)
        assert actual.shape == (rows, n), (rows, n, k)
        try:
            assert_matches_f32_reference(actual, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k))
        except AssertionError as error:
            raise AssertionError(f"rows={rows} n={n} k={k}: {error}") from error


@pytest.mark.parametrize("n,k", [(96, 512), (72, 1024), (50, 768), (35, 512)])
@pytest.mark.parametrize("qname", tuple(QTYPES))
def test_grouped_decode_matches_oracle(ops, oracle, qname, n, k):
    """(K of two to four super-blocks: 4, 4, 2 and 1 weight rows per pass-long row for these four shapes)"""
    tgo, _, synth = ops
    qtype, experts = QTYPES[qname], 40
    host = synth.random_packed_weight(qtype, (experts, n), k, seed=400 + qtype)
    sizes = [1, 1, 2, 1, 9, 1, 3, 1, 1, 8, 1, 1, 2, 1, 1, 1]          # 34 rows over 16 groups
    chosen = [0, 3, 4, 7, 9, 12, 13, 17, 20, 21, 25, 28, 30, 33, 36, 39]
    offsets = np.cumsum(sizes).tolist()
    x = random_bf16((offsets[-1], k), seed=23)
    indices = torch.tensor(chosen, device="cuda", dtype=torch.int64)
    ends = torch.tensor(offsets, device="cuda", dtype=torch.int32)
    actual = tgo.grouped_mmq(x, host.cuda(), indices, ends, qtype, n)
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), chosen, offsets, n, k, n)
    assert_matches_f32_reference(actual, exact)

    second = synth.random_packed_weight(qtype, (experts, n), k, seed=500 + qtype)
    out_first, out_second = tgo.grouped_mmq_pair(x, host.cuda(), second.cuda(), indices, ends, qtype, n)
    torch.testing.assert_close(out_first, actual, rtol=0, atol=0)
    exact_second = oracle.grouped(oracle.mmq_forward, qtype, bits(x), second.numpy(), chosen, offsets, n, k, n)
    assert_matches_f32_reference(out_second, exact_second)


def test_grouped_decode_skips_invalid_groups(ops, oracle):
    tgo, _, synth = ops
    qtype, n, k = 14, 48, 256
    host = synth.random_packed_weight(qtype, (6, n), k, seed=9)
    x = random_bf16((8, k), seed=29)
    chosen, offsets = [1, 11, 2, 3], [2, 4, 4, 8]      # group 1: unknown expert, group 2: empty
    actual = tgo.grouped_mmq(
        x, host.cuda(), torch.tensor(chosen, device="cuda"), torch.tensor(offsets, device="cuda", dtype=torch.int32), qtype, n
    )
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), chosen, offsets, n, k, n)
    covered = ~np.isnan(exact[:, 0])
    assert covered.sum() == 6
    assert_matches_f32_reference(actual[torch.from_numpy(covered).cuda()], exact[covered])


@pytest.mark.parametrize("qname", ("IQ2_S", "Q5_K"))
def test_skewed_small_batch_listed_with_every_expert(ops, oracle, qname):
    """256 listed experts, one group of 200 rows and a few single rows: the host sees 256 rows over 256 groups and
    takes the bandwidth kernel, which walks the large group eight rows at a time (its tasks share the expert's weights
    through the L2: measured 29 us against 52 us for the matrix-core kernel on the same call with only the non-empty
    groups listed; one group has to reach about 500 rows before the matrix-core kernel wins, and a call of that many
    rows over few listed groups takes it anyway).  Results match the oracle either way."""
    tgo, native, synth = ops
    qtype, n, k, experts = QTYPES[qname], 96, 512, 256
    sizes = [0] * experts
    sizes[7] = 200
    for expert in (3, 40, 41, 200, 255):
        sizes[expert] = 1
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    assert native.lib.tgo_forward_kernel_family(rows, experts) == b"gemv"
    host = synth.random_packed_weight(qtype, (experts, n), k, seed=321 + qtype)
    x = random_bf16((rows, k), seed=12)
    indices = torch.arange(experts, dtype=torch.int64, device="cuda")
    actual = tgo.grouped_mmq(x, host.cuda(), indices, torch.tensor(offsets, dtype=torch.int32, device="cuda"), qtype, n)
    expected = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), list(range(experts)), offsets, n, k, n)
    assert_matches_f32_reference(actual, expected)
    # the same rows with only the non-empty groups listed take the matrix-core kernel
    listed = [e for e in range(experts) if sizes[e] > 0]
    assert native.lib.tgo_forward_kernel_family(rows, len(listed)) == b"mfma"
    compact = tgo.grouped_mmq(x, host.cuda(), torch.tensor(listed, dtype=torch.int64, device="cuda"),
                              torch.tensor(np.cumsum([sizes[e] for e in listed]).tolist(), dtype=torch.int32, device="cuda"), qtype, n)
    assert_matches_f32_reference(compact, expected)


@pytest.mark.parametrize("experts", (700, 1500))
@pytest.mark.parametrize("qname", ("IQ2_S", "Q6_K", "Q3_K"))
def test_grouped_decode_finds_tasks_among_many_groups(ops, oracle, qname, experts):
    """Small grouped calls of these formats are one launch whose workgroups look their task up in the group list
    themselves, 256 groups per round: 700 listed groups (nearly all empty, some with more than one task, some naming an
    expert that does not exist) make the lookup run three rounds, with tasks on both sides of every round's boundary.
    (1500 listed groups are more than that launch accepts: the same call with the task list built by one workgroup.)"""
    tgo, native, synth = ops
    qtype, n, k = QTYPES[qname], 40, 512
    rng = np.random.default_rng(77 + qtype)
    sizes = np.zeros(experts, dtype=np.int64)
    for group, size in ((0, 9), (100, 1), (254, 2), (255, 3), (256, 1), (257, 8), (300, 4), (511, 2), (512, 10),
                        (513, 1), (600, 5), (699, 3)):
        sizes[group] = size
    chosen = rng.permutation(experts)
    unknown = [100, 255, 300, 513]
    chosen[unknown] = [experts, experts + 7, -1, 10**9]
    offsets = np.cumsum(sizes).tolist()
    rows = offsets[-1]
    assert rows <= 64 and native.lib.tgo_forward_kernel_family(rows, experts) == b"gemv"
    host = synth.random_packed_weight(qtype, (experts, n), k, seed=55 + qtype)
    x = random_bf16((rows, k), seed=19)
    actual = tgo.grouped_mmq(x, host.cuda(), torch.tensor(chosen, dtype=torch.int64, device="cuda"),
                             torch.tensor(offsets, dtype=torch.int32, device="cuda"), qtype, n)
    exact = oracle.grouped(oracle.mmq_forward, qtype, bits(x), host.numpy(), chosen.tolist(), offsets, n, k, n)
    covered = ~np.isnan(exact[:, 0])
    assert covered.sum() == rows - sum(int(sizes[g]) for g in unknown)
    assert_matches_f32_reference(actual[torch.from_numpy(covered).cuda()], exact[covered])


@pytest.mark.parametrize("qname", ("IQ2_S", "Q6_K", "Q3_K"))
@pytest.mark.parametrize("rows", (15, 64, 72))
def test_one_launch_and_two_launch_decode_agree(ops, qname, rows):
    """Calls of at most 8 (dense) or 64 (grouped) rows quantize inside the decode kernels, larger ones in a launch of
    their own; the arithmetic is the same, so a call split into small ones gives the same bits."""
    tgo, _, synth = ops
    qtype, n, k, experts = QTYPES[qname], 48, 2304, 24
    weight = synth.random_packed_weight(qtype, (experts, n), k, seed=61 + qtype).cuda()
    x = random_bf16((rows, k), seed=rows)
    sizes = np.full(experts, rows // experts)
    sizes[: rows % experts] += 1
    indices = torch.arange(experts, dtype=torch.int64, device="cuda")
    whole = tgo.grouped_mmq(x, weight, indices, torch.tensor(np.cumsum(sizes), dtype=torch.int32, device="cuda"), qtype, n)
    begin = 0
    for expert, size in enumerate(sizes.tolist()):
        if size == 0:   # (an empty group is legal, a dense call without rows is not)
            continue
        part = tgo.mmq(x[begin:begin + size].clone(), weight[expert].clone(), qtype, n)
        torch.testing.assert_close(whole[begin:begin + size], part, rtol=0, atol=0)
        begin += size


@pytest.mark.parametrize("qname", ("IQ2_S", "Q6_K"))
def test_gathered_decode_reads_absent_rows_as_zeros(ops, qname):
    """The decode kernels that quantize their own activations gather them too: an index outside the token range is a
    row of zeros, and every other row equals the plain call on the gathered rows bit for bit."""
    tgo, _, synth = ops
    qtype, n, k = QTYPES[qname], 48, 2304
    weight = synth.random_packed_weight(qtype, (3, n), k, seed=41).cuda()
    hidden = random_bf16((4, k), seed=42)
    row_index = torch.tensor([2, -1, 0, 9, 3, 1], device="cuda", dtype=torch.int64)
    indices = torch.tensor([0, 2], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([2, 6], device="cuda", dtype=torch.int32)
    out = tgo.grouped_mmq_gathered(hidden, row_index, weight, indices, offsets, qtype, n)
    padded = torch.cat([hidden, torch.zeros_like(hidden[:1])])
    safe = torch.tensor([2, 4, 0, 4, 3, 1], device="cuda")
    expected = tgo.grouped_mmq(padded.index_select(0, safe), weight, indices, offsets, qtype, n)
    torch.testing.assert_close(out, expected, rtol=0, atol=0)
    assert torch.count_nonzero(out[1]) == 0 and torch.count_nonzero(out[3]) == 0
