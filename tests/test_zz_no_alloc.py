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
