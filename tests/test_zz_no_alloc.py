"""paras_moe_route_noalloc: the routing entry point that allocates nothing (its
scratch is a fixed array in the library's device image).  Checked against
paras_moe_route through the C ABI, bit for bit, on two calls in a row of which
the second is smaller (the array keeps the first call's contents), against
the oracle, and for its size limits."""
import pytest
import torch

import capi
import oracle as O
from conftest import assert_bit_exact

pytestmark = pytest.mark.gpu
NAMES = ("topi", "topw", "order", "inv", "counts", "offsets")


def test_two_calls_in_a_row_match_the_workspace_entry_point():
    torch.manual_seed(11)
    for T, E, k, dtype in [(8192, 8, 2, torch.bfloat16), (777, 8, 2, torch.bfloat16)]:
        logits = torch.randn(T, E).to(dtype)
        if T > 10:
            logits[3] = logits[3, 0]          # every expert tied
        dl = logits.cuda()
        want = capi.moe_route(dl, k)
        got = capi.moe_route_noalloc(dl, k)
        for name, g, w in zip(NAMES, got, want):
            assert_bit_exact(g, w, f"noalloc vs workspace entry point: {name} T{T}")
        for name, g, w in zip(NAMES, got, O.moe_route(logits, k)):
            assert_bit_exact(g, w, f"noalloc vs oracle: {name} T{T}")


def test_more_experts_other_dtypes_and_the_largest_input():
    torch.manual_seed(12)
    for T, E, k, dtype in [(65536, 8, 2, torch.bfloat16), (300, 64, 8, torch.float32), (5000, 3, 3, torch.float16), (1, 8, 2, torch.bfloat16)]:
        dl = torch.randn(T, E).to(dtype).cuda()
        want = capi.moe_route(dl, k)
        got = capi.moe_route_noalloc(dl, k)
        for name, g, w in zip(NAMES, got, want):
            assert_bit_exact(g, w, f"{name} T{T} E{E} k{k}")


def test_allocates_nothing_and_rejects_what_does_not_fit():
    dl = torch.randn(4096, 8).bfloat16().cuda()
    out = capi.moe_route_noalloc(dl, 2)           # first call on the device done: the symbol address is resolved
    torch.cuda.synchronize()
    L = capi.lib()
    import ctypes as C
    a0, c0 = C.c_uint64(), C.c_uint64()
    L.paras_memory_stats(0, C.byref(a0), C.byref(c0))
    before = torch.cuda.memory_stats()["num_alloc_retries"], torch.cuda.memory_allocated()
    free0 = torch.cuda.mem_get_info()[0]          # what the driver itself has left: a direct hipMalloc would show here
    capi.moe_route_noalloc(dl, 2, out=out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    a1, c1 = C.c_uint64(), C.c_uint64()
    L.paras_memory_stats(0, C.byref(a1), C.byref(c1))
    assert (a0.value, c0.value) == (a1.value, c1.value)
    assert before == (torch.cuda.memory_stats()["num_alloc_retries"], torch.cuda.memory_allocated())
    # under stream capture an allocation (or a free) would fail the capture; replays give the same outputs
    want = [o.clone() for o in out]
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            capi.moe_route_noalloc(dl, 2, out=out)
    for _ in range(3):
        for o in out:
            o.zero_()
        g.replay()
        torch.cuda.synchronize()
        for name, got, w in zip(NAMES, out, want):
            assert_bit_exact(got, w, f"replayed {name}")
    with pytest.raises(capi.ParasError, match="exceed the static scratch"):
        capi.moe_route_noalloc(torch.zeros(65537, 8, device="cuda"), 2)
    with pytest.raises(capi.ParasError, match="expert count"):
        capi.moe_route_noalloc(torch.zeros(16, 65, device="cuda"), 2)
    with pytest.raises(capi.ParasError, match="at least one token"):
        capi.moe_route_noalloc(torch.zeros(0, 8, device="cuda"), 2)
