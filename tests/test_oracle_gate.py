"""Pins the gate oracle (/root/reference/comfy/ldm/hidream/model.py:263-283): the fixed-order C restatement
against torch's library kernels, an fp64 brute force and exact small-integer cases."""
import itertools
import math

import torch
import torch.nn.functional as F

from oracle import hidream_moe_oracle as O

BF16 = torch.bfloat16


def rand_gate(T, D, E, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, D), generator=g).to(BF16)
    wg = (torch.randn((E, D), generator=g) / math.sqrt(D)).to(BF16)
    return x, wg


def test_top2_rule_all_orderings_with_ties():
    vals = [0.1, 0.2, 0.3, 0.4]
    rows = torch.tensor(list(itertools.product(vals, repeat=4)))          # includes every tie pattern
    idx, w = O.top2_lowest_index(rows)
    for r, i in zip(rows.tolist(), idx.tolist()):
        want = sorted(range(4), key=lambda e: (-r[e], e))[:2]
        assert i == want


def test_fixed_order_exact_on_integer_inputs():
    # small integers: every partial sum is exact in fp32 whatever the order, so all three evaluations of the
    # logits must agree exactly, and with them scores' order and the routing
    g = torch.Generator().manual_seed(3)
    T, D, E = 200, 512, 4
    x = torch.randint(-3, 4, (T, D), generator=g).float().to(BF16)
    wg = (torch.randint(-2, 3, (E, D), generator=g).float() / 64).to(BF16)
    idx, w, logits, scores = O.gate_fixed_order(x, wg)
    exact = (x.double() @ wg.double().t())
    assert torch.equal(logits.double(), exact.to(BF16).double())
    ti, tw, tl, ts = O.gate_torch(x, wg)
    assert torch.equal(tl.view(torch.int16), logits.view(torch.int16))
    sm = torch.softmax(logits.double(), dim=-1)
    assert float((scores.double() - sm).abs().max()) <= 2 ** -9          # bf16 rounding of a value <= 1
    same_scores = (scores.view(torch.int16) == ts.view(torch.int16)).all(dim=1)
    assert float(same_scores.float().mean()) > 0.98                      # exp() differs by an fp32 ulp at most
    assert torch.equal(idx[same_scores].long(), ti[same_scores])
    # ties that survive bf16 rounding go to the lower index
    srt = torch.sort(scores.float(), dim=-1, descending=True, stable=True).indices[:, :2]
    assert torch.equal(idx.long(), srt)


def test_fixed_order_vs_torch_and_fp64_on_random_inputs():
    T, D, E = 4096, 2560, 4
    x, wg = rand_gate(T, D, E, 0)
    idx, w, logits, scores = O.gate_fixed_order(x, wg)
    ti, tw, tl, ts = O.gate_torch(x, wg)
    l64 = x.double() @ wg.double().t()
    # (1) bf16 logits: equal to the rounding of the fp64 value unless that value sits closer to a rounding midpoint
    # than fp32 summation can resolve (2^-27 of the sum of |terms|; observed <= 2e-9 of it) -- "fragile" logits
    lo = l64.to(BF16)
    bits = lo.view(torch.int16).to(torch.int32)
    up = (bits + 1).to(torch.int16).view(BF16).double()       # neighbours of the rounded value (same sign side
    dn = (bits - 1).to(torch.int16).view(BF16).double()       # handling is irrelevant: only the distance matters)
    mid_a, mid_b = (lo.double() + up) / 2, (lo.double() + dn) / 2
    dist_to_mid = torch.minimum((l64 - mid_a).abs(), (l64 - mid_b).abs())
    sumabs = x.double().abs() @ wg.double().abs().t()
    fragile = dist_to_mid <= sumabs * 2 ** -27
    assert float(fragile.float().mean()) < 2e-3
    for name, lg in (("fixed-order", logits), ("torch", tl)):
        bad = (lg.view(torch.int16) != lo.view(torch.int16)) & ~fragile
        assert int(bad.sum()) == 0, (name, int(bad.sum()))
    # (2) routing: identical on every token whose bf16 logits agree between the two evaluations and whose scores
    # agree; the others must be few
    tok_same = (logits.view(torch.int16) == tl.view(torch.int16)).all(dim=1) & \
               (scores.view(torch.int16) == ts.view(torch.int16)).all(dim=1)
    assert float(tok_same.float().mean()) > 0.99
    assert torch.equal(idx[tok_same].long(), ti[tok_same])
    assert torch.equal(w[tok_same].view(torch.int16), tw[tok_same].view(torch.int16))
    # (3) against torch.topk (what the reference calls) on tie-free rows
    tk_w, tk_i = torch.topk(ts, k=2, dim=-1, sorted=False)
    s_sorted = torch.sort(ts.float(), dim=-1, descending=True).values
    tie_free = (s_sorted[:, 0] != s_sorted[:, 1]) & (s_sorted[:, 1] != s_sorted[:, 2])
    assert float(tie_free.float().mean()) > 0.98
    a = torch.sort(tk_i[tie_free], dim=-1).values
    b = torch.sort(ti[tie_free], dim=-1).values
    assert torch.equal(a, b)
    # (4) weights are the selected scores, not renormalised (norm_topk_prob False, model.py:253,278)
    assert torch.equal(w.view(torch.int16), torch.gather(scores, 1, idx.long()).view(torch.int16))
    assert float((w.float().sum(dim=1)).max()) <= 1.0 + 2 ** -7


def test_softmax_known_answers():
    D, E = 512, 4
    wg = torch.zeros((E, D), dtype=BF16)
    x = torch.zeros((2, D), dtype=BF16)
    idx, w, logits, scores = O.gate_fixed_order(x, wg)
    assert idx.tolist() == [[0, 1], [0, 1]] and scores.float().tolist() == [[0.25] * 4] * 2
    # logits (ln 3, 0, 0, ln 1/3 ...) -> closed-form softmax
    wg[0, 0], wg[3, 0] = 1.0, -1.0
    x[:, 0] = 2.0
    idx, w, logits, scores = O.gate_fixed_order(x, wg)
    e = [math.exp(2.0), 1.0, 1.0, math.exp(-2.0)]
    want = torch.tensor([v / sum(e) for v in e]).to(BF16).float()
    assert torch.equal(scores[0].float(), want)
    assert idx[0].tolist() == [0, 1]           # experts 1 and 2 tie exactly -> lower index


def test_generic_D_and_E():
    for (T, D, E, seed) in [(33, 264, 16, 1), (50, 1024, 2, 2), (20, 2568, 8, 3)]:
        x, wg = rand_gate(T, D, E, seed)
        idx, w, logits, scores = O.gate_fixed_order(x, wg)
        ref = (x.double() @ wg.double().t())
        assert float((logits.double() - ref).abs().max()) <= float(ref.abs().max()) * 2 ** -7
        srt = torch.sort(scores.float(), dim=-1, descending=True, stable=True).indices[:, :2]
        assert torch.equal(idx.long(), srt)


def test_renorm_topk_rounding_points_and_closed_forms():
    """model.py:277-280 on bf16 tensors: equal weights give exactly one half each; the result is the fp64 quotient
    within the rounding of the bf16 sum and of the bf16 quotient; all-zero weights stay zero (the 1e-20 guard)."""
    g = torch.Generator().manual_seed(3)
    w = torch.rand((4096, 2), generator=g).to(torch.bfloat16)
    w[::7, 1] = w[::7, 0]
    w[5] = 0
    r = O.renorm_topk(w)
    assert r.dtype == torch.bfloat16
    eq = w[:, 0] == w[:, 1]
    nz = w[:, 0] != 0
    assert bool((r[eq & nz].float() == 0.5).all())
    assert bool((r[5].float() == 0).all())
    # explicit rounding points
    s = (w[:, 0].float() + w[:, 1].float()).to(torch.bfloat16)
    d = (s.float() + 1e-20).to(torch.bfloat16)
    want = (w.float() / d.float().unsqueeze(-1)).to(torch.bfloat16)
    assert torch.equal(r.view(torch.int16), want.view(torch.int16))
    exact = w.double() / (w.double().sum(-1, keepdim=True) + 1e-20)
    ok = nz
    assert float(((r.double() - exact).abs()[ok] / exact[ok].clamp_min(1e-3)).max()) < 3 * 2.0 ** -8


# ---- the same gate on fp16 tensors (the Hunyuan3D block's other dtype) ----------------------------------------

F16 = torch.float16


def test_f16_conversions_of_the_checker_equal_torch():
    """The C checker's fp16 decode on all 65536 patterns and its encode on random values, every representable
    value, every midpoint between neighbours (ties to even), the overflow boundary and the subnormal range, against
    torch's own conversion."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    dec = O.f16_decode(bits)
    want = bits.view(F16).float()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(dec), nan)
    assert torch.equal(dec[~nan].view(torch.int32), want[~nan].view(torch.int32))      # incl. the sign of zero
    g = torch.Generator().manual_seed(0)
    finite = want[~nan & ~torch.isinf(want)]
    pos = torch.sort(finite[finite >= 0]).values
    mids = ((pos[:-1].double() + pos[1:].double()) / 2).float()                         # exact in fp32
    vals = torch.cat([
        torch.randn(200000, generator=g) * 10.0 ** torch.randint(-9, 6, (200000,), generator=g).float(),
        finite, mids, -mids,
        torch.tensor([65504.0, 65519.0, 65519.996, 65520.0, 65536.0, 1e9, float("inf"), -float("inf"), -65520.0,
                      2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 1.5 * 2.0 ** -24, 2.5 * 2.0 ** -24, 2.0 ** -14,
                      0.0, -0.0, 1e-30]),
    ])
    enc = O.f16_encode(vals)
    assert torch.equal(enc, vals.to(F16).view(torch.int16))
    assert O.f16_encode(torch.tensor([float("nan")])).view(F16).isnan().all()


def test_fixed_order_f16_vs_torch_and_fp64():
    """fp16 gate: logits equal the fp16 rounding of the fp64 value except where that value sits on a rounding
    midpoint to within what fp32 summation resolves; routing equal to torch's own fp16 kernels wherever logits and
    scores agree bit for bit; small-integer inputs exact; ties to the lower index."""
    T, D, E = 2048, 2048, 8
    g = torch.Generator().manual_seed(5)
    x = torch.randn((T, D), generator=g).to(F16)
    wg = (torch.randn((E, D), generator=g) / math.sqrt(D)).to(F16)
    idx, w, logits, scores = O.gate_fixed_order(x, wg)
    assert w.dtype == F16 and logits.dtype == F16
    ti, tw, tl, ts = O.gate_torch(x, wg)
    l64 = x.double() @ wg.double().t()
    lo = l64.to(F16)
    bits = lo.view(torch.int16).to(torch.int32)
    up = (bits + 1).to(torch.int16).view(F16).double()
    dn = (bits - 1).to(torch.int16).view(F16).double()
    dist_to_mid = torch.minimum((l64 - (lo.double() + up) / 2).abs(), (l64 - (lo.double() + dn) / 2).abs())
    sumabs = x.double().abs() @ wg.double().abs().t()
    fragile = dist_to_mid <= sumabs * 2 ** -26             # observed <= 1e-8 of the sum of |terms|
    assert float(fragile.float().mean()) < 2e-2            # fp16 has 8x finer steps than bf16: more midpoints nearby
    bad = (logits.view(torch.int16) != lo.view(torch.int16)) & ~fragile
    assert int(bad.sum()) == 0
    tok_same = (logits.view(torch.int16) == tl.view(torch.int16)).all(dim=1) & \
               (scores.view(torch.int16) == ts.view(torch.int16)).all(dim=1)
    assert float(tok_same.float().mean()) > 0.9
    assert torch.equal(idx[tok_same].long(), ti[tok_same])
    assert torch.equal(w[tok_same].view(torch.int16), tw[tok_same].view(torch.int16))
    sm = torch.softmax(logits.double(), dim=-1)
    assert float((scores.double() - sm).abs().max()) <= 2 ** -12          # fp16 rounding of a value <= 1
    assert torch.equal(w.view(torch.int16), torch.gather(scores, 1, idx.long()).view(torch.int16))
    srt = torch.sort(scores.float(), dim=-1, descending=True, stable=True).indices[:, :2]
    assert torch.equal(idx.long(), srt)
    # small integers: exact whatever the order
    xi = torch.randint(-3, 4, (100, 512), generator=g).float().to(F16)
    wi = (torch.randint(-2, 3, (4, 512), generator=g).float() / 64).to(F16)
    _, _, li, si = O.gate_fixed_order(xi, wi)
    assert torch.equal(li.double(), (xi.double() @ wi.double().t()).to(F16).double())
    # all-zero logits: scores 0.25 each, experts 0 and 1
    i0, w0, _, s0 = O.gate_fixed_order(torch.zeros((2, 512), dtype=F16), torch.zeros((4, 512), dtype=F16))
    assert i0.tolist() == [[0, 1], [0, 1]] and s0.float().tolist() == [[0.25] * 4] * 2
