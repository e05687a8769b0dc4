"""The entry point that allocates nothing: tgo_mmq_forward_static against tgo_mmq_forward (-m gpu).

Both are called through the C ABI on the same seeded inputs; the static variant keeps its q8_1 activation
workspace in a fixed per-GPU array of the library and must return the same bits, also on a second, smaller call
that finds the first call's contents in that array, for the GEMV-sized and the MFMA-sized regime alike.
"""

import numpy as np
import pytest
import torch

from helpers import QTYPES, assert_matches_f32_reference, bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def native():
    import torch_ggml_ops  # noqa: F401
    import synth
    from torch_ggml_ops import _native

    assert torch.cuda.is_available()
    return _native, synth


def _forward(native, x, packed, n, qtype, static):
    lib = native.lib
    rows, k = x.shape
    out = torch.full((rows, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        native.check(lib.tgo_mmq_forward_static(x.data_ptr(), packed.data_ptr(), out.data_ptr(), rows, k, n, qtype, stream))
    else:
        workspace = torch.empty(lib.tgo_q8_workspace_bytes(rows, k), dtype=torch.uint8, device="cuda")
        native.check(lib.tgo_mmq_forward(x.data_ptr(), packed.data_ptr(), out.data_ptr(), workspace.data_ptr(), rows, k, n, qtype, stream))
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("qname", ("Q4_K", "IQ2_S"))
def test_static_workspace_forward_equals_the_workspace_argument_form(native, oracle, qname):
    _native, synth = native
    qtype, n, k = QTYPES[qname], 200, 1024
    host = synth.random_packed_weight(qtype, (n,), k, seed=610 + qtype)
    packed = host.cuda()
    generator = torch.Generator(device="cuda").manual_seed(61)
    # a call that fills many tiles of the array, then smaller ones that find its contents there:
    # MFMA-sized with a ragged last tile, GEMV-sized, a single row
    for rows in (300, 77, 8, 1):
        x = torch.randn(rows, k, device="cuda", generator=generator).to(torch.bfloat16)
        expected = _forward(_native, x, packed, n, qtype, static=False)
        actual = _forward(_native, x, packed, n, qtype, static=True)
        np.testing.assert_array_equal(bits(actual), bits(expected), err_msg=f"{qname} rows={rows}")
        if rows <= 8:
            assert_matches_f32_reference(actual, oracle.mmq_forward(qtype, bits(x), host.numpy(), n, k))


def test_static_workspace_rejects_what_does_not_fit(native):
    _native, _ = native
    lib = _native.lib
    buffer = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = buffer.data_ptr()
    rows, k = 4096, 2048   # 10.5 MB of q8_1 blocks
    assert lib.tgo_q8_workspace_bytes(rows, k) > 4 * 1024 * 1024
    assert lib.tgo_mmq_forward_static(p, p, p, rows, k, 8, 12, None) == 1
    assert b"static workspace" in lib.tgo_last_error()


def test_static_workspace_forward_leaves_device_memory_alone(native):
    """The driver's count of free device memory is the same before and after calls of the static form (inputs and
    outputs allocated beforehand; the first call, which looks up the array's address, comes before the count)."""
    _native, synth = native
    lib = _native.lib
    qtype, rows, n, k = QTYPES["Q5_K"], 300, 200, 1024
    packed = synth.random_packed_weight(qtype, (n,), k, seed=7).cuda()
    x = torch.randn(rows, k, device="cuda").to(torch.bfloat16)
    out = torch.empty(rows, n, dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    _native.check(lib.tgo_mmq_forward_static(x.data_ptr(), packed.data_ptr(), out.data_ptr(), rows, k, n, qtype, stream))
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for smaller in (rows, 77, 1):
        _native.check(lib.tgo_mmq_forward_static(x.data_ptr(), packed.data_ptr(), out.data_ptr(), smaller, k, n, qtype, stream))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
