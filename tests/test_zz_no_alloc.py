"""The entry point that allocates nothing: llmq_backward_bias_bf16_static_scratch keeps its band sums in an
array built into the library's device code instead of a caller-provided scratch buffer.  Its results must equal
llmq_backward_bias_bf16's bit for bit (same kernels, same fixed summation order), on two calls in a row of which
the second is smaller (the shared array keeps the first call's contents), and it must refuse shapes whose band
sums exceed the array.  Called through the C ABI."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

LIMIT = 16 << 20   # LLMQ_BACKWARD_BIAS_STATIC_SCRATCH_BYTES in include/llmq_fp8.h


def _run_both(capi, dout, fmt, start, sa, sb, BT, OC):
    st = torch.cuda.current_stream().cuda_stream
    need = int(capi.lib.llmq_backward_bias_scratch_bytes(BT, OC, fmt))
    assert 0 < need <= LIMIT
    scratch = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    want = start.clone()
    capi.check(capi.lib.llmq_backward_bias_bf16(want.data_ptr(), dout.data_ptr(), fmt, sa.data_ptr(), sb.data_ptr(),
                                                scratch.data_ptr(), need, BT, OC, st))
    got = start.clone()
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0])
    capi.check(capi.lib.llmq_backward_bias_bf16_static_scratch(got.data_ptr(), dout.data_ptr(), fmt, sa.data_ptr(),
                                                               sb.data_ptr(), BT, OC, st))
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]) == before   # nothing allocated, by torch or by HIP
    return got.view(torch.int16).cpu().numpy(), want.view(torch.int16).cpu().numpy()


@pytest.mark.parametrize("fmt", [0, 1, 2], ids=["e4m3", "e5m2", "bf16"])
def test_static_scratch_matches_caller_scratch_twice(fmt):
    from llmq_amd import capi
    g = torch.Generator(device="cuda").manual_seed(11 + fmt)
    sa = torch.tensor([0.375], device="cuda")
    sb = torch.tensor([1.5], device="cuda")
    # first a large call, then a smaller one with different band / column counts: the second must not see
    # anything the first left in the shared array
    for BT, OC in [(8192, 4608), (1000, 1152)]:
        if fmt == 2:
            dout = torch.randn((BT, OC), device="cuda", generator=g).to(torch.bfloat16)
        else:
            codes = torch.randint(0, 256, (BT, OC), device="cuda", dtype=torch.uint8, generator=g)
            codes = torch.where((codes & 0x7C) == 0x7C, codes ^ 0x40, codes)   # no NaN / Inf codes in either format
            dout = codes
        start = torch.randn(OC, device="cuda", generator=g).to(torch.bfloat16)
        got, want = _run_both(capi, dout, fmt, start, sa, sb, BT, OC)
        assert np.array_equal(got, want), (BT, OC)
        assert not np.array_equal(got, start.view(torch.int16).cpu().numpy())


def test_static_scratch_rejects_oversized_shape():
    from llmq_amd import capi
    BT, OC = 64, 5 << 20                     # one band of 5 Mi columns: 20 MiB of band sums
    assert int(capi.lib.llmq_backward_bias_scratch_bytes(BT, OC, 0)) > LIMIT
    p = torch.zeros(16, dtype=torch.uint8, device="cuda").data_ptr()   # never dereferenced: the call is refused first
    rc = capi.lib.llmq_backward_bias_bf16_static_scratch(p, p, 0, None, None, BT, OC, None)
    assert rc == capi.LLMQ_ERR_INVALID_ARGUMENT
    assert b"built-in scratch" in capi.lib.llmq_last_error()


def test_static_scratch_entry_replays_from_a_hip_graph():
    """After one ordinary call on the device (the first call looks up the built-in array's address, a host-side
    query), the entry point is two kernel launches and nothing else: captured into a HIP graph and replayed three
    times with eager work in between, every replay must equal the eager result bit for bit."""
    from llmq_amd import capi
    BT, OC, fmt = 4096, 2304, 0
    g = torch.Generator(device="cuda").manual_seed(5)
    codes = torch.randint(0, 256, (BT, OC), device="cuda", dtype=torch.uint8, generator=g)
    dout = torch.where((codes & 0x7F) == 0x7F, codes ^ 0x40, codes)          # no NaN codes
    sa, sb = torch.tensor([0.5], device="cuda"), torch.tensor([0.25], device="cuda")
    start = torch.randn(OC, device="cuda", generator=g).to(torch.bfloat16)

    def call(dbias):
        capi.check(capi.lib.llmq_backward_bias_bf16_static_scratch(dbias.data_ptr(), dout.data_ptr(), fmt, sa.data_ptr(),
                                                                   sb.data_ptr(), BT, OC, torch.cuda.current_stream().cuda_stream))

    want = start.clone()
    call(want)                                   # the eager call every capture must be preceded by
    torch.cuda.synchronize()
    got = start.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(got)
    for _ in range(3):
        got.copy_(start)
        other = start.clone()
        call(other)                              # eager use of the same array between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        assert torch.equal(other.view(torch.int16), want.view(torch.int16))
