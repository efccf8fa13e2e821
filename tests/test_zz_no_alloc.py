"""ccf_route_static, the entry point that allocates nothing, against ccf_route.

Two calls in a row through the C ABI, the second with a smaller input: the
built-in scratch keeps the first call's contents, and every result of both
calls must equal ccf_route's bit for bit.  Sizes beyond the built-in scratch
are rejected with an error code.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

KEYS = ("counts", "offsets", "pos", "src_row", "dst_row", "inv_pos", "idx_kept")


def _idx(n, E, seed, dropped=0.0):
    g = torch.Generator().manual_seed(seed)
    # skewed ids so that a capacity limit binds on some experts
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -1.2
    idx = torch.multinomial(p / p.sum(), n, replacement=True, generator=g)
    if dropped:
        idx[torch.rand(n, generator=g) < dropped] = -1
    return idx.to(torch.int64)


def _compare(n, E, k, cap, seed):
    from ccfuser_amd import ops
    idx = _idx(n, E, seed, dropped=0.05).cuda()
    ref = ops.route(idx, E, k, cap)
    got = ops.route_static(idx, E, k, cap)
    torch.cuda.synchronize()
    R = int(ref["offsets"][-1])
    assert R == int(got["offsets"][-1])
    for key in ("counts", "offsets", "inv_pos", "idx_kept"):
        assert torch.equal(ref[key], got[key]), key
    for key in ("pos", "src_row", "dst_row"):                  # first R entries are defined
        assert torch.equal(ref[key][:R], got[key][:R]), key


def test_two_calls_second_smaller_match_route():
    _compare(50_000, 32, 2, 2_000, seed=11)      # 49 chunks x 32 experts, capacity binds
    _compare(3_000, 8, 2, -1, seed=12)           # 3 chunks x 8 experts over the first call's leftovers
    _compare(1, 1, 1, -1, seed=13)


def _outputs(n, E):
    dev = "cuda"
    return {
        "counts": torch.empty(E, dtype=torch.int32, device=dev),
        "offsets": torch.empty(E + 1, dtype=torch.int32, device=dev),
        "pos": torch.empty(n, dtype=torch.int64, device=dev),
        "src_row": torch.empty(n, dtype=torch.int32, device=dev),
        "dst_row": torch.empty(n, dtype=torch.int32, device=dev),
        "inv_pos": torch.empty(n, dtype=torch.int32, device=dev),
        "idx_kept": torch.empty(n, dtype=torch.int64, device=dev),
    }


def test_the_call_allocates_no_device_memory_and_can_be_captured():
    """What the entry point exists for: with the outputs allocated beforehand the C call leaves
    the device's free memory and torch's reserved memory where they were (both the small-table
    path and the one with a scan launch, 1024 experts, which also sets an LDS attribute), and a
    warmed-up call can be recorded into a HIP graph whose replays, with fresh inputs, equal
    ccf_route bit for bit."""
    from ccfuser_amd import ops
    for n, E, k, cap, seed in ((20_000, 16, 2, 1_500, 21), (40_000, 1024, 1, -1, 22)):
        idx = _idx(n, E, seed).cuda()
        out = _outputs(n, E)
        ops.route_static(idx, E, k, cap, out=out)            # first use on this device: looks the scratch address up
        torch.cuda.synchronize()
        free0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        for _ in range(3):
            ops.route_static(idx, E, k, cap, out=out)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_reserved() == reserved0
        ref = ops.route(idx, E, k, cap)
        R = int(ref["offsets"][-1])
        for key in KEYS:
            m = R if key in ("pos", "src_row", "dst_row") else None
            assert torch.equal(ref[key][:m], out[key][:m]), key
    # capture and replay
    n, E, k, cap = 20_000, 16, 2, 1_500
    idx_static = _idx(n, E, 31).cuda()
    out = _outputs(n, E)
    side = torch.cuda.Stream()                               # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.route_static(idx_static, E, k, cap, out=out)     # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.route_static(idx_static, E, k, cap, out=out)
    for rep in range(3):
        fresh = _idx(n, E, 40 + rep).cuda()
        ref = ops.route(fresh, E, k, cap)                    # eager work between the replays
        torch.cuda.synchronize()
        idx_static.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        R = int(ref["offsets"][-1])
        for key in KEYS:
            m = R if key in ("pos", "src_row", "dst_row") else None
            assert torch.equal(ref[key][:m], out[key][:m]), (rep, key)


def test_sizes_beyond_the_builtin_scratch_are_rejected():
    from ccfuser_amd import _lib, ops
    lib = _lib.lib()
    limit = lib.ccf_route_static_max_entries()
    assert limit == 1 << 18
    E = 1024
    n = (limit // E + 1) * 1024                  # one chunk too many for 1024 experts
    idx = torch.zeros(n, dtype=torch.int64, device="cuda")
    with pytest.raises(_lib.CcfError) as err:
        ops.route_static(idx, E, 1)
    assert err.value.code == 2 and "built-in scratch" in str(err.value)
    # the largest accepted size still works
    n_ok = (limit // E) * 1024
    got = ops.route_static(idx[:n_ok], E, 1)
    torch.cuda.synchronize()
    assert int(got["counts"][0]) == n_ok and int(got["offsets"][-1]) == n_ok
