"""HIP graph capture of the operators (-m gpu): decode loops are launch-bound, so callers capture them.

The operators allocate through torch's caching allocator, launch on the current stream and never
synchronise, which is all a capture needs.  Each replay is checked against the eager result, with eager
work and synchronisations between the replays.
"""

import pytest
import torch

from helpers import QTYPES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch_ggml_ops
    import synth

    assert torch.cuda.is_available()
    return torch_ggml_ops, synth


def _capture(fn):
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        outputs = fn()
    return graph, outputs


def test_decode_layer_replays_bit_identically(ops):
    tgo, synth = ops
    experts, tokens = 64, 4
    gate = synth.random_packed_weight(QTYPES["IQ2_S"], (experts, 512), 2048, 11, device="cuda")
    up = synth.random_packed_weight(QTYPES["IQ2_S"], (experts, 512), 2048, 12, device="cuda")
    down = synth.random_packed_weight(QTYPES["Q6_K"], (experts, 2048), 512, 13, device="cuda")
    token_of_row, indices, offsets, _ = synth.zipf_routing(tokens, experts, 8, 7, device="cuda")
    generator = torch.Generator(device="cuda").manual_seed(3)
    hidden = torch.randn(tokens, 2048, device="cuda", generator=generator).to(torch.bfloat16)
    x = hidden.index_select(0, token_of_row).contiguous()

    def layer():
        gate_rows, up_rows = tgo.grouped_mmq_pair(x, gate, up, indices, offsets, QTYPES["IQ2_S"], 512)
        activated = torch.nn.functional.silu(gate_rows) * up_rows
        return tgo.grouped_mmq(activated, down, indices, offsets, QTYPES["Q6_K"], 2048)

    eager = layer().clone()
    graph, captured = _capture(layer)
    for replay in range(4):
        captured.zero_()
        scratch = torch.randn(1 << 16, device="cuda").sum()   # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), f"replay {replay} differs from the eager result"
        assert torch.isfinite(scratch)
    # new activations in the captured input buffer give the matching new result
    fresh = torch.randn(tokens, 2048, device="cuda", generator=generator).to(torch.bfloat16)
    x.copy_(fresh.index_select(0, token_of_row))
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(captured, layer())


def test_dense_and_prefill_sized_calls_capture(ops):
    tgo, synth = ops
    qtype, n, k = QTYPES["Q4_K"], 1024, 2048
    weight = synth.random_packed_weight(qtype, (n,), k, 21, device="cuda")
    generator = torch.Generator(device="cuda").manual_seed(4)
    for rows in (1, 8, 300):   # GEMV family, its largest task, the MFMA family
        x = torch.randn(rows, k, device="cuda", generator=generator).to(torch.bfloat16)
        dy = torch.randn(rows, n, device="cuda", generator=generator).to(torch.bfloat16)

        def step():
            return tgo.mmq(x, weight, qtype, n), torch.ops.torch_ggml_ops.mmq_grad_input.default(dy, weight, qtype, k)

        eager = [t.clone() for t in step()]
        graph, captured = _capture(step)
        for _ in range(3):
            for tensor in captured:
                tensor.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for got, expected in zip(captured, eager):
                assert torch.equal(got, expected)


def test_scaled_pair_with_short_groups_replays_bit_identically(ops):
    """A grouped pair large enough for the scaled operands, with whole groups of at most 32 rows among the others: the
    launch's trailing workgroups take those from cursors that the quantizer's launch zeroes, so every replay starts
    from a fresh count."""
    from torch_ggml_ops import _native

    tgo, synth = ops
    qtype, n, k, experts = QTYPES["Q5_K"], 512, 1024, 24
    sizes = [3000, 1, 17, 700, 32, 2500, 9, 260, 31, 1800, 5, 2, 900, 33, 1500]
    indices = torch.tensor(list(range(len(sizes)))[::-1], device="cuda", dtype=torch.int64)
    offsets = torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(device="cuda", dtype=torch.int32)
    rows = int(sum(sizes))
    assert _native.forward_operand_for(qtype, rows, n, 2) == "scaled"
    gate = synth.random_packed_weight(qtype, (experts, n), k, 31, device="cuda")
    up = synth.random_packed_weight(qtype, (experts, n), k, 32, device="cuda")
    generator = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(rows, k, device="cuda", generator=generator).to(torch.bfloat16)

    def pair():
        return tgo.grouped_mmq_pair(x, gate, up, indices, offsets, qtype, n)

    eager = [t.clone() for t in pair()]
    graph, captured = _capture(pair)
    for replay in range(4):
        for t in captured:
            t.zero_()
        scratch = torch.randn(1 << 16, device="cuda").sum()   # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {replay} differs from the eager result"
        assert torch.isfinite(scratch)


def test_launch_stream_is_torch_current_stream(ops):
    """The handle the operators launch on is that of torch's current stream, on the default stream and inside
    ``torch.cuda.stream(...)``; the device context is only entered when another device is current."""
    from torch_ggml_ops import _native

    device = torch.device("cuda", torch.cuda.current_device())
    assert _native.stream_of(device) == torch.cuda.current_stream(device).cuda_stream
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert _native.stream_of(device) == side.cuda_stream
    assert _native.stream_of(device) == torch.cuda.current_stream(device).cuda_stream
    with _native.on_device(device):
        assert torch.cuda.current_device() == device.index
    assert _native.stream_of(torch.device("cuda")) == torch.cuda.current_stream().cuda_stream   # no index: torch's own call
