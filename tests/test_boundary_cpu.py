"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports every symbol
declared in include/tgo.h, its argument checks fire before any launch, the Python
validators reproduce the reference's error contract (message fragments of
tests/test_mmq.py:176-223 and tests/test_grouped_mmq.py:483-561 in the reference), and the
operators' fake kernels / schemas are registered.  No kernel is launched here.
"""

import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def package():
    import torch_ggml_ops
    import synth
    from torch_ggml_ops import _native, _validate

    return torch_ggml_ops, _native, _validate, synth


def test_library_exports_every_declared_symbol(package):
    _, native, _, _ = package
    header = (ROOT / "include" / "tgo.h").read_text()
    declared = set(re.findall(r"\b(tgo_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found in include/tgo.h"
    for name in sorted(declared):
        assert hasattr(native.lib, name), f"{name} is declared but not exported"
    assert declared == set(native.EXPORTS)


def test_sizes_and_block_bytes(package):
    _, native, _, synth = package
    lib = native.lib
    assert lib.tgo_version() >= 110   # (the workspace grew with the scaled operands: callers size it through the library)
    for qtype, size in synth.BLOCK_BYTES.items():
        assert lib.tgo_block_bytes(qtype) == size
    assert lib.tgo_block_bytes(10) == 0
    # two bytes per value (fp16 operands) + two fp32 per 32 values + a power of two and 16 bytes of block sums per 256
    # values + a power of two per row, rows padded to 32, plus the 1 KiB tail
    assert lib.tgo_q8_workspace_bytes(33, 512) == 2 * 64 * 512 + 2 * 64 * 16 * 4 + 64 * 2 * (4 + 16) + 64 * 4 + 1024
    assert lib.tgo_q8_workspace_bytes(0, 512) == 0
    # the kind a call would use: scaled once it has 128 tiles of 256 rows x 128 outputs (both projections count)
    assert native.forward_operand() == "auto"
    assert native.forward_operand_for(13, 4096, 1024, 1) == "scaled"
    assert native.forward_operand_for(13, 4096, 1024 - 128, 1) == "int8"
    assert native.forward_operand_for(22, 512, 4096, 1) == "half"
    assert native.forward_operand_for(22, 2048, 1024, 2) == "scaled"
    assert lib.tgo_task_workspace_bytes(100, 7) % 16 == 0
    assert lib.tgo_task_workspace_bytes(100, 7) >= 4 * (1 + 3 * (13 + 7))


def test_c_abi_rejects_bad_arguments_before_launch(package):
    _, native, _, _ = package
    lib = native.lib
    fake = 0x10000  # never dereferenced: every call below fails its checks first
    assert lib.tgo_mmq_forward(fake, fake, fake, fake, 0, 256, 8, 12, None) == 1
    assert b"zero-row" in lib.tgo_last_error()
    assert lib.tgo_mmq_forward(fake, fake, fake, fake, 4, 300, 8, 12, None) == 1
    assert b"multiple of 256" in lib.tgo_last_error()
    assert lib.tgo_mmq_forward(fake, fake, fake, fake, 4, 256, 8, 10, None) == 1
    assert b"unsupported quant_type" in lib.tgo_last_error()
    assert lib.tgo_mmq_forward(fake, fake + 2, fake, fake, 4, 256, 8, 12, None) == 1
    assert b"16-byte aligned" in lib.tgo_last_error()
    assert lib.tgo_mmq_grad_input(None, fake, fake, fake, 4, 8, 256, 12, None) == 1
    assert b"must not be null" in lib.tgo_last_error()
    assert lib.tgo_grouped_mmq_forward(fake, fake, None, fake, None, fake, fake, fake, 4, 256, 8, 2, 3, 12, None) == 1
    assert b"active expert count exceeds" in lib.tgo_last_error()
    assert lib.tgo_grouped_mmq_forward(fake, fake, fake, fake, None, fake, fake, fake, 4, 256, 8, 4, 3, 12, None) == 1
    assert b"given together" in lib.tgo_last_error()
    total, count = ctypes.c_double(), ctypes.c_int64()
    assert lib.tgo_profile_read(99, ctypes.byref(total), ctypes.byref(count)) == 1


def test_dense_validation_messages(package):
    _, _, validate, synth = package
    validate.REQUIRE_DEVICE = False
    try:
        packed = synth.random_packed_weight(12, (37,), 2048, seed=1)
        x = torch.randn(4, 2048).to(torch.bfloat16)
        assert validate.dense(x, packed, 12, 37, backward=False) == (4, 2048, 37)
        assert validate.dense(torch.randn(2, 3, 37).to(torch.bfloat16), packed, 12, 2048, backward=True) == (6, 2048, 37)
        cases = [
            (lambda: validate.dense(x[:, ::2], packed, 12, 37, backward=False), "contiguous"),
            (lambda: validate.dense(x[1:], packed, 12, 37, backward=False), "zero storage offset"),
            (lambda: validate.dense(x, packed.reshape(-1)[:-1].clone(), 12, 37, backward=False), "expected"),
            (lambda: validate.dense(x, packed, 10, 37, backward=False), "unsupported quant_type"),
            (lambda: validate.dense(x[:0], packed, 12, 37, backward=False), "zero-row"),
            (lambda: validate.dense(x.float(), packed, 12, 37, backward=False), "torch.bfloat16"),
            (lambda: validate.dense(x, packed.to(torch.int8), 12, 37, backward=False), "torch.uint8"),
            (lambda: validate.dense(x[:, :300].contiguous(), packed, 12, 37, backward=False), "multiple of 256"),
            (lambda: validate.dense(x, packed, 12, 0, backward=False), "out_features must be positive"),
            (lambda: validate.dense(x[:, :37].contiguous(), packed, 12, 2000, backward=True), "multiple of 256"),
            (lambda: validate.dense(x[:0, :37].contiguous(), packed, 12, 2048, backward=True), "zero-row"),
        ]
        for call, fragment in cases:
            with pytest.raises(RuntimeError, match=fragment):
                call()
    finally:
        validate.REQUIRE_DEVICE = True
    with pytest.raises(RuntimeError, match="CUDA/HIP tensor"):
        validate.dense(x, packed, 12, 37, backward=False)


def test_grouped_validation_messages(package):
    _, _, validate, synth = package
    validate.REQUIRE_DEVICE = False
    try:
        packed = synth.random_packed_weight(12, (8, 37), 2048, seed=2)
        x = torch.randn(262, 2048).to(torch.bfloat16)
        experts = torch.tensor([0, 2, 5, 7], dtype=torch.int64)
        offsets = torch.tensor([1, 128, 257, 262], dtype=torch.int32)
        shape = validate.grouped(x, packed, experts, offsets, 12, 37, backward=False)
        assert shape == (262, 2048, 37, 8, 4, 37 * 8 * 144)
        cases = [
            (lambda: validate.grouped(x[:, ::2], packed, experts, offsets, 12, 37, backward=False), "contiguous"),
            (lambda: validate.grouped(x[1:], packed, experts, offsets, 12, 37, backward=False), "zero storage offset"),
            (lambda: validate.grouped(x, packed[:, :, :-1].contiguous(), experts, offsets, 12, 37, backward=False), "bytes per row"),
            (lambda: validate.grouped(x, packed, experts, offsets, 10, 37, backward=False), "unsupported quant_type"),
            (lambda: validate.grouped(x[:0], packed, experts, offsets, 12, 37, backward=False), "zero-row"),
            (lambda: validate.grouped(x, packed, experts, offsets.long(), 12, 37, backward=False), "torch.int32"),
            (lambda: validate.grouped(x, packed, experts.int(), offsets, 12, 37, backward=False), "torch.int64"),
            (lambda: validate.grouped(x, packed, experts[:3], offsets, 12, 37, backward=False), "equal lengths"),
            (lambda: validate.grouped(x, packed[0], experts, offsets, 12, 37, backward=False), r"\[experts, out_features, row_bytes\]"),
            (lambda: validate.grouped(x, packed, experts, offsets, 12, 38, backward=False), "does not match out_features"),
            (lambda: validate.grouped(x, packed[:3].contiguous(), experts, offsets, 12, 37, backward=False), "active expert count exceeds"),
            (lambda: validate.grouped(x[:, :37].contiguous(), packed, experts, offsets, 12, 2000, backward=True), "multiple of 256"),
        ]
        for call, fragment in cases:
            with pytest.raises(RuntimeError, match=fragment):
                call()
    finally:
        validate.REQUIRE_DEVICE = True


def test_second_weight_of_a_pair_is_checked_like_the_first(package):
    """A second weight with the first one's geometry needs no second pass through the checks; any other goes through
    them and fails with their message (or with the pair's own, when it is a valid weight of another expert count)."""
    from torch_ggml_ops.grouped_mmq import _forward

    _, _, validate, synth = package
    validate.REQUIRE_DEVICE = False
    try:
        packed = synth.random_packed_weight(12, (8, 37), 2048, seed=2)
        other = synth.random_packed_weight(12, (8, 37), 2048, seed=3)
        assert validate.same_weight_geometry(packed, other)
        assert not validate.same_weight_geometry(packed, other[:, :, :-1])                  # not contiguous
        assert not validate.same_weight_geometry(packed, other[:4].contiguous())           # fewer experts
        assert not validate.same_weight_geometry(packed, other.to(torch.int8))             # another dtype
        assert not validate.same_weight_geometry(packed, other.reshape(-1)[16:].reshape(-1))   # another shape, offset
        x = torch.randn(262, 2048).to(torch.bfloat16)
        experts = torch.tensor([0, 2, 5, 7], dtype=torch.int64)
        offsets = torch.tensor([1, 128, 257, 262], dtype=torch.int32)
        cases = [
            (other[:, :, :-1], "contiguous"),
            (other[:, :36].contiguous(), "does not match out_features"),
            (other.to(torch.int8), "torch.uint8"),
            (other[:4].contiguous(), "identical physical geometry"),
        ]
        for second, fragment in cases:
            with pytest.raises(RuntimeError, match=fragment):
                _forward(x, packed, second, experts, offsets, 12, 37)
    finally:
        validate.REQUIRE_DEVICE = True


def test_operator_schemas_and_fake_kernels(package):
    tgo, _, _, _ = package
    ops = torch.ops.torch_ggml_ops
    assert str(ops.mmq.default._schema) == (
        "torch_ggml_ops::mmq(Tensor input, Tensor packed_weight, int quant_type, int out_features) -> Tensor"
    )
    assert "-> (Tensor, Tensor)" in str(ops.grouped_mmq_pair.default._schema)
    x = torch.empty(3, 5, 512, dtype=torch.bfloat16, device="meta")
    w = torch.empty(37, 288, dtype=torch.uint8, device="meta")
    assert tgo.mmq(x, w, 12, 37).shape == (3, 5, 37)
    assert ops.mmq_grad_input.default(torch.empty(3, 5, 37, dtype=torch.bfloat16, device="meta"), w, 12, 512).shape == (3, 5, 512)
    rows = torch.empty(20, 512, dtype=torch.bfloat16, device="meta")
    experts = torch.empty(8, 37, 288, dtype=torch.uint8, device="meta")
    indices = torch.empty(4, dtype=torch.int64, device="meta")
    offsets = torch.empty(4, dtype=torch.int32, device="meta")
    assert tgo.grouped_mmq(rows, experts, indices, offsets, 12, 37).shape == (20, 37)
    first, second = tgo.grouped_mmq_pair(rows, experts, experts, indices, offsets, 12, 37)
    assert first.shape == second.shape == (20, 37)
    grad = torch.empty(20, 37, dtype=torch.bfloat16, device="meta")
    assert ops.grouped_mmq_grad_input.default(grad, experts, indices, offsets, 12, 512).shape == (20, 512)
    assert ops.grouped_mmq_pair_grad_input.default(grad, grad, experts, experts, indices, offsets, 12, 512).shape == (20, 512)


def test_cpu_tensors_have_no_fallback(package):
    tgo, _, _, synth = package
    packed = synth.random_packed_weight(12, (4,), 256, seed=3)
    x = torch.randn(2, 256).to(torch.bfloat16)
    with pytest.raises(NotImplementedError):
        tgo.mmq(x, packed, 12, 4)


def test_synthetic_generators_are_seeded_and_well_formed(package, oracle):
    _, _, _, synth = package
    import numpy as np

    for qtype in synth.BLOCK_BYTES:
        first = synth.random_packed_weight(qtype, (3, 5), 512, seed=11)
        again = synth.random_packed_weight(qtype, (3, 5), 512, seed=11)
        assert torch.equal(first, again) and first.shape == (3, 5, synth.row_bytes(qtype, 512))
        values = oracle.dequant_f32(qtype, first.numpy(), 512)
        assert np.isfinite(values).all()
    tokens, indices, offsets, weights = synth.zipf_routing(64, 16, 4, seed=5)
    assert tokens.numel() == 256 == int(offsets[-1]) and weights.numel() == 256
    assert (indices[1:] > indices[:-1]).all() and (offsets[1:] > offsets[:-1]).all()


def test_token_runs_drop_rows_outside_the_input(package):
    """The host half of the per-token sum behind the gathered operators' gradients: the rows listed token by token in
    row order, with the rows whose index lies outside the token range behind the last run (the kernel that adds the
    runs up never sees them).  Summing the runs on the CPU gives the per-token sums."""
    from torch_ggml_ops.gathered import _token_runs

    grad_rows = torch.arange(24, dtype=torch.float32).reshape(6, 4).to(torch.bfloat16)
    row_index = torch.tensor([2, -1, 0, 9, 3, 2])
    order, starts = _token_runs(row_index, 4)
    assert order.dtype == torch.int64 and starts.dtype == torch.int64
    assert starts.tolist() == [0, 1, 1, 3, 4]
    assert order.tolist()[:4] == [2, 0, 5, 4] and sorted(order.tolist()[4:]) == [1, 3]
    result = torch.zeros(4, 4)
    for token in range(4):
        for row in order[starts[token]:starts[token + 1]].tolist():
            result[token] += grad_rows[row].float()
    expected = torch.zeros(4, 4)
    for row, token in enumerate(row_index.tolist()):
        if 0 <= token < 4:
            expected[token] += grad_rows[row].float()
    torch.testing.assert_close(result, expected, rtol=0, atol=0)
