"""GGUF container reader against files assembled by hand from the published layout.

No GGUF file ships with the reference (its tests point at an external checkpoint) and the ``gguf`` package
it reads them with is not installed, so the reader is pinned on the container specification itself: the
test writes every field with explicit ``struct.pack`` calls (magic, version, counts, typed metadata, tensor
infos, alignment padding, data) and checks what the reader returns field by field.  Agreement with the
``gguf`` package on a real checkpoint is therefore not pinned.
"""

import struct

import numpy as np
import pytest
import torch

from torch_ggml_ops.gguf_file import GGML_BLOCK, GGUFError, GGUFReader, load_packed_tensor


def _string(text: str) -> bytes:
    raw = text.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


def _kv(key: str, value_type: int, payload: bytes) -> bytes:
    return _string(key) + struct.pack("<I", value_type) + payload


def _assemble(tensors, metadata=(), version=3, alignment=None, misalign=None):
    """tensors: list of (name, ggml dims, ggml type, bytes).  Returns (file bytes, data offsets)."""
    fields = list(metadata)
    if alignment is not None:
        fields.append(_kv("general.alignment", 4, struct.pack("<I", alignment)))
    align = alignment or 32
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(fields)) + b"".join(fields)
    infos, blobs, offset, offsets = b"", b"", 0, []
    for name, dims, tensor_type, payload in tensors:
        stored = offset + (misalign or 0)
        infos += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", tensor_type, stored)
        offsets.append(stored)
        padded = payload + b"\0" * (-len(payload) % align)
        blobs += padded
        offset += len(padded)
    head += infos
    head += b"\0" * (-len(head) % align)
    return head + blobs, offsets


def _random_bytes(count, seed):
    return np.random.default_rng(seed).integers(0, 256, count, dtype=np.uint8).tobytes()


def test_reads_metadata_and_tensor_table(tmp_path):
    q4k = _random_bytes(2 * 5 * 144, 1)            # dims (256, 5, 2): two experts of five rows
    q6k = _random_bytes(3 * 2 * 210, 2)            # dims (512, 3)
    iq2s = _random_bytes(7 * 82, 3)                # dims (256, 7)
    f32 = np.arange(12, dtype=np.float32)
    bf16 = np.arange(8, dtype=np.uint16)
    metadata = [
        _kv("general.architecture", 8, _string("qwen3moe")),
        _kv("u8", 0, struct.pack("<B", 200)), _kv("i8", 1, struct.pack("<b", -3)),
        _kv("u16", 2, struct.pack("<H", 60000)), _kv("i16", 3, struct.pack("<h", -300)),
        _kv("u32", 4, struct.pack("<I", 4000000000)), _kv("i32", 5, struct.pack("<i", -7)),
        _kv("f32", 6, struct.pack("<f", 0.5)), _kv("flag", 7, struct.pack("<?", True)),
        _kv("u64", 10, struct.pack("<Q", 2**40)), _kv("i64", 11, struct.pack("<q", -(2**40))),
        _kv("f64", 12, struct.pack("<d", 1e-300)),
        _kv("ints", 9, struct.pack("<IQ", 5, 3) + struct.pack("<3i", 1, -2, 3)),
        _kv("names", 9, struct.pack("<IQ", 8, 2) + _string("a") + _string("größe")),
    ]
    tensors = [
        ("blk.0.ffn_gate_exps.weight", (256, 5, 2), 12, q4k),
        ("blk.0.attn_v.weight", (512, 3), 14, q6k),
        ("blk.0.ffn_down.weight", (256, 7), 22, iq2s),
        ("norm.weight", (4, 3), 0, f32.tobytes()),
        ("half.weight", (8,), 30, bf16.tobytes()),
    ]
    blob, offsets = _assemble(tensors, metadata, alignment=64)
    path = tmp_path / "model.gguf"
    path.write_bytes(blob)

    with GGUFReader(path) as reader:
        assert reader.version == 3 and reader.alignment == 64 and reader.data_offset % 64 == 0
        fields = reader.fields
        assert fields["general.architecture"] == "qwen3moe"
        assert (fields["u8"], fields["i8"], fields["u16"], fields["i16"]) == (200, -3, 60000, -300)
        assert (fields["u32"], fields["i32"], fields["flag"]) == (4000000000, -7, True)
        assert (fields["u64"], fields["i64"], fields["f32"], fields["f64"]) == (2**40, -(2**40), 0.5, 1e-300)
        assert fields["ints"] == [1, -2, 3] and fields["names"] == ["a", "größe"]

        assert [t.name for t in reader.tensors] == [t[0] for t in tensors]
        gate = reader.get_tensor("blk.0.ffn_gate_exps.weight")
        assert gate.tensor_type == 12 and gate.type_name == "Q4_K" and gate.shape == (256, 5, 2)
        assert gate.n_elements == 2560 and gate.n_bytes == len(q4k)
        assert gate.data.dtype == np.uint8 and gate.data.shape == (2, 5, 144)
        assert gate.data.tobytes() == q4k
        assert gate.data_offset == reader.data_offset + offsets[0]
        assert blob[gate.data_offset:gate.data_offset + 16] == q4k[:16]

        value = reader.get_tensor("blk.0.attn_v.weight")
        assert value.data.shape == (3, 2 * 210) and value.data.tobytes() == q6k
        down = reader.get_tensor("blk.0.ffn_down.weight")
        assert down.data.shape == (7, 82) and down.data.tobytes() == iq2s and down.type_name == "IQ2_S"
        norm = reader.get_tensor("norm.weight")
        assert norm.data.dtype == np.float32 and norm.data.shape == (3, 4)
        assert np.array_equal(norm.data, f32.reshape(3, 4))
        half = reader.get_tensor("half.weight")
        assert half.data.dtype == np.uint16 and np.array_equal(half.data, bf16)
        with pytest.raises(KeyError):
            reader.get_tensor("missing")

        host = load_packed_tensor(gate, "cpu")
        assert host.dtype == torch.uint8 and host.is_contiguous() and tuple(host.shape) == (2, 5, 144)
        assert host.numpy().tobytes() == q4k
        with pytest.raises(GGUFError, match="not a block-quantized"):
            load_packed_tensor(norm, "cpu")


def test_version_2_and_default_alignment(tmp_path):
    payload = _random_bytes(110, 4)
    blob, _ = _assemble([("w", (256,), 11, payload)], version=2)
    path = tmp_path / "v2.gguf"
    path.write_bytes(blob)
    with GGUFReader(path) as reader:
        assert reader.version == 2 and reader.alignment == 32 and reader.data_offset % 32 == 0
        assert reader.tensors[0].data.shape == (110,) and reader.tensors[0].data.tobytes() == payload


def test_block_table_matches_the_kernels():
    from torch_ggml_ops import _native

    for qtype in (11, 12, 13, 14, 22):
        assert GGML_BLOCK[qtype] == (256, _native.lib.tgo_block_bytes(qtype))


@pytest.mark.parametrize(
    "mutate,message",
    (
        (lambda b: b"GGML" + b[4:], "magic"),
        (lambda b: b[:4] + struct.pack("<I", 1) + b[8:], "version"),
        (lambda b: b[:-40], "beyond the file"),
        (lambda b: b[:30], "truncated"),
        (lambda b: b[:10], "too small"),
    ),
)
def test_rejects_damaged_files(tmp_path, mutate, message):
    blob, _ = _assemble([("w", (256, 2), 12, _random_bytes(288, 5))])
    path = tmp_path / "bad.gguf"
    path.write_bytes(mutate(blob))
    with pytest.raises(GGUFError, match=message):
        GGUFReader(path)


def test_rejects_inconsistent_tensor_infos(tmp_path):
    path = tmp_path / "bad.gguf"
    path.write_bytes(_assemble([("w", (256,), 12, _random_bytes(144, 6))], misalign=8)[0])
    with pytest.raises(GGUFError, match="alignment"):
        GGUFReader(path)
    path.write_bytes(_assemble([("w", (100,), 12, _random_bytes(144, 6))])[0])
    with pytest.raises(GGUFError, match="multiple of the block size"):
        GGUFReader(path)
    path.write_bytes(_assemble([("w", (256,), 99, _random_bytes(144, 6))])[0])
    with pytest.raises(GGUFError, match="unknown ggml type"):
        GGUFReader(path)
    path.write_bytes(_assemble([("w", (256,), 12, _random_bytes(144, 6))], alignment=48)[0])
    with pytest.raises(GGUFError, match="power of two"):
        GGUFReader(path)


@pytest.mark.gpu
def test_file_to_device_to_grouped_operator(tmp_path):
    """Experts written to a GGUF file, read back and uploaded in chunks, give the same operator output bit for
    bit as the same bytes uploaded directly."""
    import torch_ggml_ops as tgo
    import synth

    experts, n, k, qtype = 4, 96, 512, 13
    host = synth.random_packed_weight(qtype, (experts, n), k, seed=77)
    blob, _ = _assemble([("blk.3.ffn_up_exps.weight", (k, n, experts), qtype, host.numpy().tobytes())])
    path = tmp_path / "experts.gguf"
    path.write_bytes(blob)
    with GGUFReader(path) as reader:
        tensor = reader.get_tensor("blk.3.ffn_up_exps.weight")
        assert int(tensor.shape[0]) == k
        packed = load_packed_tensor(tensor, "cuda", chunk_bytes=10000)  # several chunks, the last one partial
    assert packed.is_cuda and tuple(packed.shape) == tuple(host.shape)
    assert torch.equal(packed.cpu(), host)
    generator = torch.Generator(device="cpu").manual_seed(5)
    x = torch.randn(50, k, generator=generator).to(torch.bfloat16).cuda()
    indices = torch.tensor([0, 1, 3], device="cuda", dtype=torch.int64)
    offsets = torch.tensor([20, 21, 50], device="cuda", dtype=torch.int32)
    from_file = tgo.grouped_mmq(x, packed, indices, offsets, qtype, n)
    direct = tgo.grouped_mmq(x, host.cuda(), indices, offsets, qtype, n)
    torch.testing.assert_close(from_file, direct, rtol=0, atol=0)
