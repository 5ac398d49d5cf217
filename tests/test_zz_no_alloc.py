"""hdmoe_dispatch_static, the dispatch entry point that allocates nothing (its per-chunk histograms live in a device
array inside the library image), against hdmoe_dispatch on the same routing decisions: bit-exact, through the C ABI,
on two calls in a row of which the second is smaller, so that the shared buffer still holds the first call's
histograms when the second starts. Collected last on purpose (file name)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _routing(T, E, seed):
    g = torch.Generator().manual_seed(seed)
    first = torch.randint(0, E, (T,), generator=g)
    second = (first + torch.randint(1, E, (T,), generator=g)) % E
    return torch.stack([first, second], dim=1).to(torch.int32)


def _dispatch_static(idx, E):
    from comfyui_amd import _lib
    T = idx.shape[0]
    dev = idx.device
    counts = torch.full((E,), -1, dtype=torch.int32, device=dev)
    offsets = torch.full((E + 1,), -1, dtype=torch.int32, device=dev)
    perm = torch.full((2 * T,), -1, dtype=torch.int32, device=dev)
    inv = torch.full((2 * T,), -1, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    _lib.check(_lib.lib.hdmoe_dispatch_static(idx.data_ptr(), T, E, counts.data_ptr(), offsets.data_ptr(),
                                              perm.data_ptr(), inv.data_ptr(), stream))
    return counts, offsets, perm, inv


@pytest.mark.parametrize("sizes,E", [((8192, 1000), 4), ((150001, 4097), 5), ((40000, 33), 16), ((700, 1), 8)])
def test_static_dispatch_equals_workspace_dispatch_on_two_calls(dev, sizes, E):
    from comfyui_amd import functional as HF
    from oracle import hidream_moe_oracle as O
    for call, T in enumerate(sizes):
        idx = _routing(T, E, seed=T * 7 + E + call)
        d_idx = idx.to(dev)
        got = _dispatch_static(d_idx, E)
        want = HF.dispatch(d_idx, E)
        torch.cuda.synchronize()
        for name, a, b in zip(("counts", "offsets", "perm", "inv_perm"), got, want):
            assert torch.equal(a, b), f"call {call} (T={T}, E={E}): {name} differs from hdmoe_dispatch"
        if T <= 8192:
            for name, a, b in zip(("counts", "offsets", "perm", "inv_perm"), got, O.dispatch(idx, E)):
                assert torch.equal(a.cpu(), b), f"call {call} (T={T}, E={E}): {name} differs from the oracle"


def test_static_dispatch_allocates_nothing_and_replays_in_a_graph(dev):
    """What the entry point exists for. With inputs and outputs allocated beforehand the call leaves the device's free
    memory where it was (hipMemGetInfo around it: a hipMalloc of any size would show, the library's or the runtime's),
    and it can be captured into a HIP graph: replays on new routing decisions, with eager work in between, give what
    the eager call gives."""
    from comfyui_amd import _lib
    T, E = 5000, 6
    bufs = [torch.full((n,), -1, dtype=torch.int32, device=dev) for n in (E, E + 1, 2 * T, 2 * T)]
    routings = [_routing(T, E, seed=s).to(dev) for s in (1, 2, 3)]
    idx = routings[0].clone()
    stream = torch.cuda.current_stream(dev).cuda_stream
    call = lambda s: _lib.check(_lib.lib.hdmoe_dispatch_static(idx.data_ptr(), T, E, *[b.data_ptr() for b in bufs], s))
    call(stream)                                   # the first call on a device looks the buffer's address up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(dev)
    for _ in range(3):
        call(stream)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(dev)
    assert free1 == free0, f"device memory moved by {free0 - free1} bytes across calls that must not allocate"
    eager = []
    for r in routings:
        idx.copy_(r)
        call(stream)
        torch.cuda.synchronize()
        eager.append([b.clone() for b in bufs])
    side = torch.cuda.Stream()                     # default priority
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(2):
        for r, want in zip(routings, eager):
            idx.copy_(r)
            for b in bufs:
                b.fill_(-7)                        # the program's own eager work between replays
            graph.replay()
            torch.cuda.synchronize()
            for name, a, b in zip(("counts", "offsets", "perm", "inv_perm"), bufs, want):
                assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager call"


def test_static_dispatch_refuses_what_its_buffer_cannot_hold(dev):
    """Beyond hdmoe_dispatch_static_max_tokens(E) the call returns HDMOE_E_WORKSPACE and enqueues nothing (the outputs
    keep their bytes); a bad expert count has no limit to report (0) and is refused as a shape error. Sizes only: no
    buffer of the refused size is allocated, the entry point checks before it touches anything."""
    from comfyui_amd import _lib
    L = _lib.lib
    assert L.hdmoe_dispatch_static_max_tokens(0) == 0 and L.hdmoe_dispatch_static_max_tokens(17) == 0
    for E in (4, 16):
        limit = L.hdmoe_dispatch_static_max_tokens(E)
        assert limit >= 1 << 20
        small = torch.full((64,), 0x5A5A5A5A, dtype=torch.int32, device=dev)
        idx = _routing(8, E, seed=1).to(dev)
        args = [small.data_ptr()] * 4 + [None]
        if limit + 2048 <= (2 ** 31 - 1) // 2:
            rc = L.hdmoe_dispatch_static(idx.data_ptr(), limit + 2048, E, *args)
            assert rc == _lib.E_WORKSPACE, (E, rc, L.hdmoe_last_error())
            assert b"hdmoe_dispatch" in L.hdmoe_last_error()
        rc = L.hdmoe_dispatch_static(idx.data_ptr(), 8, 17, *args)
        assert rc == _lib.E_SHAPE
        torch.cuda.synchronize()
        assert bool((small == 0x5A5A5A5A).all()), "a refused call must not write"
