"""The allocation-free routing plan (ggq_route_plan_static: scratch in a device array inside the library) against
ggq_route_plan with a caller workspace, through the C ABI: bit-identical outputs on two calls in a row, the
second on a smaller input (the shared scratch array keeps the first call's contents), and the size limits."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _outputs(routes, experts, dev):
    return (torch.empty(routes, dtype=torch.int64, device=dev), torch.empty(routes, dtype=torch.int64, device=dev),
            torch.empty(routes, dtype=torch.int64, device=dev), torch.empty(experts, dtype=torch.int32, device=dev),
            torch.empty(experts, dtype=torch.int32, device=dev), torch.empty(experts, dtype=torch.int64, device=dev),
            torch.empty(experts, dtype=torch.int32, device=dev), torch.empty(2, dtype=torch.int32, device=dev))


def _plan_with_workspace(pkg, idx, experts):
    lib = pkg._lib.load()
    tokens, k = idx.shape
    out = _outputs(tokens * k, experts, idx.device)
    ws = torch.empty(lib.ggq_route_plan_workspace_bytes(tokens, k, experts), dtype=torch.uint8, device=idx.device)
    pkg._lib.check(lib.ggq_route_plan(idx.data_ptr(), int(idx.dtype == torch.int64), tokens, k, experts, *[t.data_ptr() for t in out],
                                      ws.data_ptr(), ws.numel(), pkg._lib.stream_handle(idx.device)))
    return out


def _plan_static(pkg, idx, experts, out):
    lib = pkg._lib.load()
    tokens, k = idx.shape
    return lib.ggq_route_plan_static(idx.data_ptr(), int(idx.dtype == torch.int64), tokens, k, experts, *[t.data_ptr() for t in out],
                                     pkg._lib.stream_handle(idx.device))


def test_static_route_plan_matches_workspace_plan_on_two_calls(pkg, dev):
    g = torch.Generator().manual_seed(19260817)
    cases = [(4096, 8, 256, torch.int64), (333, 6, 200, torch.int32)]  # the second call is smaller than the first
    for tokens, k, experts, dtype in cases:
        idx = torch.randint(0, experts, (tokens, k), generator=g, dtype=dtype).to(dev)
        want = _plan_with_workspace(pkg, idx, experts)
        got = _outputs(tokens * k, experts, dev)  # outputs exist before the call: it allocates nothing itself
        pkg._lib.check(_plan_static(pkg, idx, experts, _outputs(tokens * k, experts, dev)))  # (the first call on a device looks the array up)
        torch.cuda.synchronize()
        before_torch, before_free = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
        pkg._lib.check(_plan_static(pkg, idx, experts, got))
        torch.cuda.synchronize()
        # the driver's own count of free device memory, which a hipMalloc inside the library would lower
        assert torch.cuda.memory_allocated(dev) == before_torch and torch.cuda.mem_get_info(dev)[0] == before_free
        n_active = int(want[7][0])
        assert int(got[7][0]) == n_active and int(got[7][1]) == int(want[7][1]) == 0
        for name, a, b in zip(("sorted_ids", "permutation", "inverse", "counts", "end_offsets", "active_ids", "active_end_offsets"), got, want):
            assert torch.equal(a, b), f"{name} differs at tokens={tokens} k={k} experts={experts}"


def test_static_route_plan_reports_a_bad_id_in_a_late_chunk(pkg, dev):
    idx = torch.randint(0, 16, (2560, 8), generator=torch.Generator().manual_seed(5), dtype=torch.int64)
    idx.view(-1)[300] = 99  # chunk 1 of the sort: its flag reaches the status word through a wave vote
    got = _outputs(2560 * 8, 16, dev)
    pkg._lib.check(_plan_static(pkg, idx.to(dev), 16, got))
    assert int(got[7][1]) == 1


def test_static_route_plan_under_stream_capture(pkg, dev):
    """What the entry point is for: a caller that records a HIP graph.  One warm call (the array's address is looked up
    once per device), then the call is captured and replayed on new ids; every replay equals ggq_route_plan."""
    tokens, k, experts = 1024, 8, 64
    g = torch.Generator().manual_seed(97531)
    idx = torch.randint(0, experts, (tokens, k), generator=g, dtype=torch.int64).to(dev)
    got = _outputs(tokens * k, experts, dev)
    pkg._lib.check(_plan_static(pkg, idx, experts, got))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pkg._lib.check(_plan_static(pkg, idx, experts, got))
    for _ in range(3):
        idx.copy_(torch.randint(0, experts, (tokens, k), generator=g, dtype=torch.int64))
        graph.replay()
        torch.cuda.synchronize()
        want = _plan_with_workspace(pkg, idx, experts)
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_static_route_plan_rejects_sizes_beyond_its_scratch(pkg, dev):
    idx = torch.zeros(8, 2, dtype=torch.int64, device=dev)
    lib = pkg._lib.load()
    out = _outputs(16, 300, dev)
    assert _plan_static(pkg, idx, 257, out) == -2  # experts beyond 256
    assert b"256 experts" in lib.ggq_last_error()
    # routes beyond 262144: the sizes are checked before anything is read or launched
    rc = lib.ggq_route_plan_static(idx.data_ptr(), 1, 32769, 8, 256, *[t.data_ptr() for t in out], pkg._lib.stream_handle(dev))
    assert rc == -2 and b"262144 routes" in lib.ggq_last_error()
    assert _plan_static(pkg, idx, 4, out) == 0
    torch.cuda.synchronize()
