"""Pins the dispatch and combine restatements (/root/reference/comfy/ldm/hidream/model.py:312-324)."""
import pytest
import torch

from oracle import hidream_moe_oracle as O

BF16 = torch.bfloat16


def random_topk(T, E, seed):
    g = torch.Generator().manual_seed(seed)
    first = torch.randint(0, E, (T,), generator=g)
    second = (first + torch.randint(1, E, (T,), generator=g)) % E
    return torch.stack([first, second], dim=1)


@pytest.mark.parametrize("T,E", [(0, 4), (1, 4), (37, 4), (1000, 4), (513, 8), (129, 16), (64, 2)])
def test_dispatch_invariants_and_reference_mask_order(T, E):
    idx = random_topk(T, E, T + E)
    counts, offsets, perm, inv = O.dispatch(idx, E)
    flat = idx.reshape(-1)
    n = flat.numel()
    assert int(counts.sum()) == n
    assert torch.equal(counts.long(), torch.bincount(flat, minlength=E))
    assert offsets[0] == 0 and torch.equal(offsets[1:].long(), torch.cumsum(counts.long(), 0))
    assert torch.equal(torch.sort(perm.long()).values, torch.arange(n))            # bijection
    assert torch.equal(inv.long()[perm.long()], torch.arange(n))                   # inverse
    # the reference gathers x[flat == i] for i = 0..E-1: concatenated mask order
    mask_order = torch.cat([torch.nonzero(flat == i).flatten() for i in range(E)]) if n else torch.empty(0, dtype=torch.long)
    assert torch.equal(perm.long(), mask_order)
    # == stable sort of the flat ids
    assert torch.equal(perm.long(), torch.sort(flat, stable=True).indices)
    # a token meets an expert at most once, so token ids ascend strictly inside a segment
    for e in range(E):
        seg = perm[int(offsets[e]):int(offsets[e + 1])].long() // 2
        assert bool((seg[1:] > seg[:-1]).all())


def test_dispatch_rejects_bad_ids_and_handles_empty_experts():
    with pytest.raises(ValueError):
        O.dispatch(torch.tensor([[0, 4]]), 4)
    idx = torch.tensor([[0, 1]] * 10)
    counts, offsets, perm, inv = O.dispatch(idx, 4)
    assert counts.tolist() == [10, 10, 0, 0] and offsets.tolist() == [0, 10, 20, 20, 20]


def test_combine_matches_torch_bf16_expression_bit_for_bit():
    g = torch.Generator().manual_seed(11)
    T, D = 97, 640
    y = torch.randn((2 * T, D), generator=g).to(BF16)
    w = torch.rand((T, 2), generator=g).to(BF16)
    sh = torch.randn((T, D), generator=g).to(BF16)
    inv = torch.randperm(2 * T, generator=g).to(torch.int32)
    ys = y[inv.long()].view(T, 2, D)
    want = (ys * w.unsqueeze(-1)).sum(dim=1) + sh                                  # model.py:319,324 at bf16
    assert torch.equal(O.combine_c(y, inv, w, sh).view(torch.int16), want.view(torch.int16))
    want2 = (ys * w.unsqueeze(-1)).sum(dim=1)
    assert torch.equal(O.combine_c(y, inv, w, None).view(torch.int16), want2.view(torch.int16))


def test_combine_slot_order_invariance_and_closed_forms():
    g = torch.Generator().manual_seed(12)
    T, D = 40, 64
    y = torch.randn((2 * T, D), generator=g).to(BF16)
    w = torch.rand((T, 2), generator=g).to(BF16)
    inv = torch.arange(2 * T, dtype=torch.int32)
    a = O.combine_c(y, inv, w, None)
    swapped = inv.view(T, 2).flip(1).reshape(-1).contiguous()
    b = O.combine_c(y, swapped, w.flip(1).contiguous(), None)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # weights (1, 0) select slot 0 exactly; weights (0.5, 0.5) on equal rows give the row back
    w10 = torch.tensor([[1.0, 0.0]] * T).to(BF16)
    assert torch.equal(O.combine_c(y, inv, w10, None).view(torch.int16), y[0::2].contiguous().view(torch.int16))
    ydup = y[0::2].repeat_interleave(2, dim=0).contiguous()
    half = torch.full((T, 2), 0.5).to(BF16)
    assert torch.equal(O.combine_c(ydup, inv, half, None).view(torch.int16), y[0::2].contiguous().view(torch.int16))
