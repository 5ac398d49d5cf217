"""GPU behaviour of the operation classes and of the paths ModelPatcher exercises: Linear forwards of every
operations class, offloaded weights, weight functions (the LowVramPatch hook), replaced Parameters, and the
per-expert composition the module falls back to. Each result is checked against the CPU oracle's Linear."""
import pytest
import torch

from comfyui_amd import synth
from oracle import hidream_moe_oracle as O
from tests.helpers import oracle_params, small_layer

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
FP8 = torch.float8_e4m3fn


def close(got, ref, rel):
    m = O.error_metrics(got, ref)
    assert m["rel_rms"] <= rel, m
    return m


def make_fp8_linear(cls, K, N, seed, dev, s_in=None):
    g = torch.Generator().manual_seed(seed)
    w8, sw = synth.quantize_per_tensor(torch.randn((N, K), generator=g) * 0.02)
    lin = cls.Linear(K, N, bias=False, dtype=BF16, device=dev)
    lin.weight = torch.nn.Parameter(w8.to(dev), requires_grad=False)
    with torch.no_grad():
        lin.scale_weight.copy_(sw)
        if s_in is not None and lin.scale_input is not None:
            lin.scale_input.fill_(s_in)
    x = torch.randn((3, 50, K), generator=g).to(BF16)
    return lin, x, w8, sw


def test_plain_and_manual_cast_linear(dev):
    from comfyui_amd import ops
    g = torch.Generator().manual_seed(0)
    w = (torch.randn((512, 256), generator=g) * 0.05)
    x = torch.randn((2, 33, 256), generator=g).to(BF16)
    ref = O.linear(x, O.LinearParams(w.to(BF16)), "plain")
    lin = ops.disable_weight_init.Linear(256, 512, bias=False, dtype=BF16, device=dev)
    with torch.no_grad():
        lin.weight.copy_(w)
    y = lin(x.to(dev))
    assert y.shape == (2, 33, 512) and y.dtype == BF16
    close(y.cpu(), ref, 3e-3)
    # manual_cast: weight kept in fp32 on the CPU (offloaded), cast and copied per call
    lin2 = ops.manual_cast.Linear(256, 512, bias=False, dtype=torch.float32, device="cpu")
    with torch.no_grad():
        lin2.weight.copy_(w)
    close(lin2(x.to(dev)).cpu(), ref, 3e-3)
    assert lin2.weight.device.type == "cpu"


def test_linear_with_bias(dev):
    """operations.Linear with a bias (comfy/ops.py:103-115): bias joins the fp32 accumulator, one rounding."""
    from comfyui_amd import ops
    g = torch.Generator().manual_seed(5)
    w = (torch.randn((512, 256), generator=g) * 0.05).to(BF16)
    b = torch.randn((512,), generator=g).to(BF16)
    x = torch.randn((2, 77, 256), generator=g).to(BF16)
    ref = O.linear_bias(x, w, b)
    for cls, wdev, wdtype in ((ops.disable_weight_init, dev, BF16), (ops.manual_cast, "cpu", torch.float32)):
        lin = cls.Linear(256, 512, bias=True, dtype=wdtype, device=wdev)
        with torch.no_grad():
            lin.weight.copy_(w)
            lin.bias.copy_(b)
        y = lin(x.to(dev))
        assert y.shape == (2, 77, 512) and y.dtype == BF16
        close(y.cpu(), ref, 3e-3)
        # at most one bf16 step (summation order): |y| < 8 here, so a step is at most 2^-5
        assert float((y.cpu().float() - ref.float()).abs().max()) <= 2.0 ** -5


@pytest.mark.parametrize("s_in", [1.0, 0.37, None])
def test_fp8_linear_with_bias(dev, s_in):
    """fp8_linear with a bias (ops.py:329, 345-346), as the attention projections of a scaled-fp8 checkpoint have."""
    from comfyui_amd import ops
    cls = ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=s_in is not None, override_dtype=FP8)
    K, N = 256, 512
    g = torch.Generator().manual_seed(11)
    w8, sw = synth.quantize_per_tensor(torch.randn((N, K), generator=g) * 0.02)
    lin = cls.Linear(K, N, bias=True, dtype=BF16, device=dev)
    assert lin.bias.dtype == FP8          # the class stores every parameter in the override dtype (ops.py:383-386)
    bias = torch.randn((N,), generator=g).to(FP8).to(BF16)     # what such a parameter can hold, cast as ops.py:329 does
    lin.weight = torch.nn.Parameter(w8.to(dev), requires_grad=False)
    with torch.no_grad():
        lin.bias.copy_(bias)
        lin.scale_weight.copy_(sw)
        if s_in is not None:
            lin.scale_input.fill_(s_in)
    x = torch.randn((3, 50, K), generator=g).to(BF16)
    ref = O.linear(x, O.LinearParams(w8, sw, None if s_in is None else torch.tensor(s_in), bias), "fp8mm")
    xd = x.to(dev)
    y = lin(xd)
    assert torch.equal(xd.cpu(), x)                      # the caller's tensor is not clamped in place
    assert y.shape == (3, 50, N) and y.dtype == BF16
    close(y.cpu(), ref, 3e-3)
    # integer-valued operands make the fp32 sums exact in any order: bit-exact, bias placement included
    xi = torch.randint(-4, 5, (2, 33, K), generator=g).to(BF16)
    wi = torch.randint(-4, 5, (N, K), generator=g).float()
    lin.weight = torch.nn.Parameter(wi.to(FP8).to(dev), requires_grad=False)
    with torch.no_grad():
        lin.scale_weight.fill_(0.3)
    ref_i = O.linear(xi, O.LinearParams(wi.to(FP8), torch.tensor(0.3), None if s_in is None else torch.tensor(s_in), bias),
                     "fp8mm")
    assert torch.equal(lin(xi.to(dev)).cpu().view(torch.int16), ref_i.view(torch.int16))


def test_scaled_fp8_linear_with_fp8_matmul(dev):
    from comfyui_amd import ops
    cls = ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=True, override_dtype=FP8)
    for s_in in (1.0, 0.5):
        lin, x, w8, sw = make_fp8_linear(cls, 256, 512, 1, dev, s_in)
        ref = O.linear(x, O.LinearParams(w8, sw, torch.tensor(s_in)), "fp8mm")
        xd = x.to(dev)
        before = xd.clone()
        y = lin(xd)
        close(y.cpu(), ref, 3e-3)
        assert torch.equal(xd, before)          # the input is not modified
    # 2-D input keeps its rank (ops.py:320-322, 353-354)
    assert lin(x.to(dev)[0]).shape == (50, 512)
    # scale_input None -> clamp rule
    cls2 = ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=False, override_dtype=FP8)
    lin2, x2, w82, sw2 = make_fp8_linear(cls2, 256, 512, 2, dev)
    x2 = x2 * 300
    ref2 = O.linear(x2, O.LinearParams(w82, sw2, None), "fp8mm")
    close(lin2(x2.to(dev)).cpu(), ref2, 3e-3)


def test_scaled_fp8_linear_without_fp8_matmul(dev):
    # the dequantising branch (ops.py:405-410): scale on the weight when it is the smaller operand, else on the input
    from comfyui_amd import ops
    cls = ops.scaled_fp8_ops(fp8_matrix_mult=False, scale_input=False, override_dtype=FP8)
    lin, x, w8, sw = make_fp8_linear(cls, 256, 512, 3, dev)
    for xx in (x, x[:1, :8]):                                    # 150 rows: weight smaller; 8 rows: input smaller
        ref = O.linear(xx, O.LinearParams(w8, sw), "upcast")
        close(lin(xx.contiguous().to(dev)).cpu(), ref, 3e-3)


def test_fp8_ops_linear(dev):
    from comfyui_amd import ops
    g = torch.Generator().manual_seed(4)
    w8 = (torch.randn((512, 256), generator=g)).to(FP8)
    lin = ops.fp8_ops.Linear(256, 512, bias=False, dtype=FP8, device=dev)
    lin.weight = torch.nn.Parameter(w8.to(dev), requires_grad=False)
    lin.eval()
    x = torch.randn((40, 256), generator=g).to(BF16)
    ref = O.linear(x, O.LinearParams(w8, torch.ones(()), None), "fp8mm")
    close(lin(x.to(dev)).cpu(), ref, 3e-3)


def test_weight_function_and_offloaded_weights_in_the_layer(dev):
    """What ModelPatcher's low-vram mode does to a module: weights stay on the offload device with
    comfy_cast_weights=True and a weight_function (LowVramPatch) rewrites the weight at every forward."""
    dim = 256
    sd, x = small_layer(seed=31, dim=dim, tokens=120, weights="fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    xd = x.to(dev)
    base = m(xd).cpu()
    # (a) offload two Linears and the gate to the CPU: results unchanged
    m.experts[1].w2.to("cpu")
    m.shared_experts.w1.to("cpu")
    m.gate.to("cpu")
    off = m(xd).cpu()
    assert torch.equal(off, base)
    # (b) a weight function that swaps in another weight (what a LoRA patch amounts to)
    other = sd["experts.0.w1.weight"].to(dev)
    lin = m.experts[2].w1
    lin.weight_function = [lambda w: other.clone()]
    patched = m(xd).cpu()
    sd2 = dict(sd)
    sd2["experts.2.w1.weight"] = sd["experts.0.w1.weight"]
    idx, w, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    ref = O.moe_forward(x, oracle_params(sd2, 4), "fp8mm", gate_result=(idx, w))
    close(patched, ref, 1e-2)
    assert not torch.equal(patched, base)
    lin.weight_function = []
    # (c) ModelPatcher replaces Parameter objects (utils.set_attr_param): the next forward must see the new one
    m.experts[2].w1.weight = torch.nn.Parameter(other.clone(), requires_grad=False)
    assert torch.equal(m(xd).cpu(), patched)


def test_mixed_dtypes_use_the_composed_path(dev):
    dim = 256
    sd, x = small_layer(seed=32, dim=dim, tokens=90, weights="fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    xd = x.to(dev)
    fused = m(xd).cpu()
    # w1 and w3 of one expert disagree on scale_input -> one quantised copy cannot serve both
    with torch.no_grad():
        m.experts[0].w3.scale_input.fill_(0.5)
    assert m._collect(xd.reshape(-1, dim)) is None
    got = m(xd).cpu()
    sd2 = dict(sd)
    sd2["experts.0.w3.scale_input"] = torch.tensor(0.5)
    idx, w, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    ref = O.moe_forward(x, oracle_params(sd2, 4), "fp8mm", gate_result=(idx, w))
    close(got, ref, 1e-2)
    assert got.shape == fused.shape


@pytest.mark.parametrize("E", [2, 8])
def test_other_expert_counts(dev, E):
    dim = 256
    sd, x = small_layer(seed=40 + E, dim=dim, tokens=333, weights="fp8", num_experts=E)
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim, num_experts=E)
    y = m(x.to(dev)).cpu()
    idx, w, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    ref = O.moe_forward(x, oracle_params(sd, E), "fp8mm", gate_result=(idx, w))
    close(y, ref, 1e-2)


def test_gate_module_signature(dev):
    from comfyui_amd import hidream
    g = hidream.MoEGate(512, 4, 2, dtype=BF16, device=dev)
    with torch.no_grad():
        g.weight.normal_(0, 512 ** -0.5)
    x = torch.randn((2, 9, 512), device=dev).to(BF16)
    idx, w, aux = g(x)
    assert idx.dtype == torch.int64 and idx.shape == (18, 2) and w.dtype == BF16 and w.shape == (18, 2) and aux is None
    ridx, rw, _, _ = O.gate_fixed_order(x.cpu().reshape(-1, 512), g.weight.detach().cpu())
    assert torch.equal(idx.cpu(), ridx.long())


def test_gate_with_renormalised_weights(dev):
    """norm_topk_prob (model.py:277-280): the kernel's quotients are the oracle's bit for bit, edge values included,
    and a layer whose gate has the flag set follows the oracle with the renormalised weights."""
    from comfyui_amd import functional as HF, hidream
    g = torch.Generator().manual_seed(77)
    w = torch.rand((5001, 2), generator=g).to(BF16)
    w[::9, 1] = w[::9, 0]
    w[3] = 0
    w[4] = torch.tensor([1.0, 0.0])
    w[5] = torch.tensor([2.0 ** -126, 2.0 ** -126])
    got = HF.renorm_top2(w.to(dev)).cpu()
    assert torch.equal(got.view(torch.int16), O.renorm_topk(w).view(torch.int16))
    assert HF.renorm_top2(w[:0].to(dev)).shape == (0, 2)

    gate = hidream.MoEGate(512, 4, 2, dtype=BF16, device=dev)
    gate.norm_topk_prob = True
    with torch.no_grad():
        gate.weight.normal_(0, 512 ** -0.5)
    x = torch.randn((3, 11, 512), device=dev).to(BF16)
    idx, wn, _ = gate(x)
    ridx, rw, _, _ = O.gate_fixed_order(x.cpu().reshape(-1, 512), gate.weight.detach().cpu())
    assert torch.equal(idx.cpu(), ridx.long())
    assert torch.equal(wn.cpu().view(torch.int16), O.renorm_topk(rw).view(torch.int16))

    dim = 256
    sd, x = small_layer(seed=61, dim=dim, tokens=210, weights="fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    plain = m(x.to(dev)).cpu()
    m.gate.norm_topk_prob = True
    y = m(x.to(dev)).cpu()
    idx, w2, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    ref = O.moe_forward(x, oracle_params(sd, 4), "fp8mm", gate_result=(idx, O.renorm_topk(w2)))
    close(y, ref, 1e-2)
    assert not torch.equal(y, plain)


def test_stacked_layers_at_32768_tokens(dev):
    """Stacked sweep (benchmark configuration 4) at its full depth: 48 independent fp8 layers at 2 x 16384 tokens,
    x <- x + FFN(LayerNorm(x)) with the block's affine-free LayerNorm (model.py:393,430) so the residual stream
    stays in range. Weights are drawn on the device (the CPU generator would need minutes for 11.5 GB) and copied
    back for the oracle. Even layers take torch's LayerNorm and the plain layer; odd layers go through the block's
    one-enqueue branch with a modulation (LayerNorm + modulation inside the gate kernel, gated residual inside the
    combine), the form the benchmark of this configuration runs.

    Every layer is called with its own workspace, and what is compared is what the layer itself decided: its routing
    rows, its segment bounds and its permutation. On every layer a token subset is followed through the oracle
    (tokens are independent through the whole stack); on layers 0, 23 and 47 ALL 32768 routing rows, the counts, the
    offsets and both permutations are compared with the oracle bit for bit, and the output subset grows to 500+ tokens
    that include the rows of the last, partial tile of every expert segment for both tile heights in use at this size,
    the tile the shared expert ends in, and rows on either side of every tile boundary near a segment start."""
    from comfyui_amd import _lib, functional as HF
    T, D, L, E, B = 32768, synth.DIM, 48, 4, 2
    S = T // B
    FULL = (0, 23, 47)
    g = torch.Generator().manual_seed(99)
    x0 = torch.randn((B, S, D), generator=g).to(BF16)
    base = torch.randperm(T, generator=g)[:32].sort().values
    xd = x0.to(dev).reshape(T, D)
    ln = lambda t: torch.nn.functional.layer_norm(t.float(), (D,), eps=1e-6).to(BF16)
    worst = dict(rel_rms=0.0, max_over_rms=0.0, max_over_max=0.0)
    lay = ws = None
    for layer in range(L):
        master, _ = synth.make_weights(layer, device=dev)
        sd_dev = synth.to_state_dict(master, "fp8")
        del master
        m = synth.build_module(sd_dev, "fp8", dev)
        sd = {k: v.cpu() for k, v in sd_dev.items()}
        branch = layer % 2 == 1
        full = layer in FULL
        wdt, experts, shared, keep = m._collect(xd)
        H, Hs = m.experts[0].w1.weight.shape[0], m.shared_experts.w1.weight.shape[0]
        if lay is None:
            lay = HF.layer_layout(T, D, H, Hs, E, _lib.W_E4M3FN)
            ws = torch.empty(lay.total, dtype=torch.uint8, device=dev)
        ws[:lay.a].fill_(0x5A)    # stale routing and permutation bytes: everything compared below must be rewritten
        x_in = xd
        if branch:
            gm = torch.Generator().manual_seed(1000 + layer)
            shift, scale = ((torch.randn((B, D), generator=gm) * 0.1).to(BF16) for _ in range(2))
            gate_mlp = (1.0 + torch.randn((B, D), generator=gm) * 0.1).to(BF16)
            out, idx_d, w_d = HF.moe_ffn(x_in, m.gate.device_weight(x_in), experts, shared, H, Hs, wdt, workspace=ws,
                                         want_routing=True, uniform_scale_in=m._uniform_scale_in,
                                         modulation=(shift.to(dev), scale.to(dev), gate_mlp.to(dev)), tokens_per_batch=S)
            xd = out
        else:
            hd = ln(x_in)
            out, idx_d, w_d = HF.moe_ffn(hd, m.gate.device_weight(hd), experts, shared, H, Hs, wdt, workspace=ws,
                                         want_routing=True, uniform_scale_in=m._uniform_scale_in)
            xd = x_in + out
        assert bool(torch.isfinite(xd.float()).all()), f"layer {layer}: non-finite residual stream"
        ints = lambda off, n: ws[off:off + 4 * n].view(torch.int32).cpu()
        offsets_d, perm_d = ints(lay.offsets, E + 1), ints(lay.perm, 2 * T)
        idx_d, w_d = idx_d.cpu(), w_d.cpu()

        def normed(rows):
            """Residual-stream rows and layer-input rows of tokens `rows` (ascending). The oracle starts every layer from
            the device's own residual stream: rounding differences of one layer would otherwise flip e4m3 neighbours in
            the next. In the branch form the LayerNorm + modulation are the library's and the oracle restates them."""
            xs = x_in[rows.to(dev)].cpu()
            if not branch:
                return xs, hd[rows.to(dev)].cpu()   # torch's LayerNorm is the harness's, not the library's: taken as is
            parts = []
            for b in range(B):
                r = xs[(rows >= b * S) & (rows < (b + 1) * S)]
                if r.shape[0]:
                    parts.append(O.ln_modulate_c(r, shift[b:b + 1], scale[b:b + 1], r.shape[0]))
            return xs, torch.cat(parts)

        sel = base
        if full:
            # routing of every token, and the dispatch it implies, against the oracle
            _, h_all = normed(torch.arange(T))
            idx_r, w_r, _, _ = O.gate_fixed_order(h_all, sd["gate.weight"])
            assert torch.equal(idx_d, idx_r), f"layer {layer}: routing indices differ"
            assert torch.equal(w_d.view(torch.int16), w_r.view(torch.int16)), f"layer {layer}: routing weights differ"
            counts_r, offs_r, perm_r, inv_r = O.dispatch(idx_r, E)
            assert torch.equal(ints(lay.counts, E), counts_r.to(torch.int32))
            assert torch.equal(offsets_d, offs_r.to(torch.int32))
            assert torch.equal(perm_d, perm_r.to(torch.int32)), f"layer {layer}: permutation differs"
            assert torch.equal(ints(lay.inv_perm, 2 * T), inv_r.reshape(-1).to(torch.int32))
            del h_all
            offs = offsets_d.tolist()
            picks = [base, torch.randperm(T, generator=g)[:160], torch.arange(T - 72, T), torch.arange(0, 24),
                     torch.arange(S - 12, S + 12),
                     torch.arange((T // 320) * 320 - 8, (T // 320) * 320 + 8), torch.arange(T - 256 - 8, T - 256 + 8)]
            for e in range(E):
                lo, hi = offs[e], offs[e + 1]
                for tile in (256, 320):
                    tail = lo + ((hi - lo) // tile) * tile          # first row of the segment's partial tile
                    rows = torch.cat([torch.arange(max(lo, tail - 8), min(hi, tail + 24)), torch.arange(max(lo, hi - 24), hi),
                                      torch.arange(lo, min(hi, lo + 12)), torch.arange(min(hi, lo + tile - 6), min(hi, lo + tile + 6))])
                    picks.append(perm_d[rows].long() // 2)
            sel = torch.unique(torch.cat(picks))
            assert sel.numel() >= 500
        xs, h = normed(sel)
        idx, w, _, _ = O.gate_fixed_order(h, sd["gate.weight"])
        assert torch.equal(idx_d[sel], idx) and torch.equal(w_d[sel].view(torch.int16), w.view(torch.int16)), layer
        y = O.moe_forward(h.unsqueeze(0), oracle_params(sd, E), "fp8mm", gate_result=(idx, w)).reshape(-1, D)
        if branch:
            b_of = (sel // S).long()
            ref = gate_mlp[b_of] * y + xs      # model.py:432-433 on bf16 tensors: product rounded, then the sum
        else:
            ref = xs + y
        got = xd[sel.to(dev)].cpu()
        met = O.error_metrics(got, ref)
        worst = {k: max(worst[k], met[k]) for k in worst}
        if layer % 8 == 0 or full:
            print(f"layer {layer} ({'branch' if branch else 'plain'}, {sel.numel()} tokens): "
                  f"rms(x)={float(got.float().pow(2).mean().sqrt()):.3f} {met}", flush=True)
        assert met["rel_rms"] <= 1e-2 and met["max_over_max"] <= 3e-2 and met["max_over_rms"] <= 3e-2, (layer, met)
        del m, sd_dev, sd, keep
    print("worst over the stack", worst)


@pytest.mark.parametrize("weights", ["fp8", "bf16"])
@pytest.mark.parametrize("rows", [1, 300, 1025])
def test_dense_swiglu_ffn(dev, weights, rows):
    """FeedForwardSwiGLU on its own (shared expert / text-token feed-forward): one quantise + two GEMM launches."""
    dim = 512
    sd, _ = small_layer(seed=50, dim=dim, tokens=8, weights=weights)
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, weights, dev, dim=dim)
    g = torch.Generator().manual_seed(rows)
    x = torch.randn((rows, dim), generator=g).to(BF16)
    ffn = m.shared_experts
    y = ffn(x.to(dev))
    assert y.shape == x.shape and y.dtype == BF16
    params = oracle_params(sd, 4)
    ref = O.ffn_swiglu(x, params["shared"], "fp8mm" if weights == "fp8" else "plain")
    close(y.cpu(), ref, 1e-2 if weights == "fp8" else 4e-3)
    # the per-Linear composition gives the same result
    y2 = ffn.w2(__import__("comfyui_amd").functional.silu_mul(ffn.w1(x.to(dev)), ffn.w3(x.to(dev))))
    close(y2.cpu(), y.cpu(), 3e-3)
    # 3-D input keeps its shape
    assert ffn(x.to(dev).view(1, rows, dim)).shape == (1, rows, dim)


def test_layer_is_graph_capturable(dev):
    """The library allocates nothing, never synchronises and issues no memsets, so a forward can be captured into a
    HIP graph. Replays (with the program's own eager work in between) must reproduce the eager result exactly."""
    dim = 512
    sd, x = small_layer(seed=60, dim=dim, tokens=600, weights="fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    xs = [x.to(dev), (x * 0.5).to(dev), x.flip(1).contiguous().to(dev)]
    eager = [m(v).clone() for v in xs]          # also warms up: kernel attributes set, scale cache filled
    torch.cuda.synchronize()
    static_x = xs[0].clone()
    side = torch.cuda.Stream()                  # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        m(static_x)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = m(static_x)
    for rep in range(2):
        for v, want in zip(xs, eager):
            static_x.copy_(v)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want)
            assert torch.equal(m(v), want)      # eager work between replays


def test_checkpoint_file_onto_the_device_and_forward(dev, tmp_path):
    """A scaled-fp8 .safetensors file is read tensor by tensor onto the GPU; the modules built from it take the
    one-call fp8 path and match the oracle run on the same file's tensors."""
    import os
    from safetensors.torch import save_file
    from comfyui_amd import checkpoint as C
    from tests.test_gpu_layer import check_layer
    pre = "model.diffusion_model."
    layer = pre + "double_stream_blocks.0.block.ff_i"
    sd, x = small_layer(seed=31, dim=512, tokens=300, weights="fp8")
    full = {f"{layer}.{k}": v for k, v in sd.items()}
    full[pre + "scaled_fp8"] = C.scaled_fp8_marker(torch.float8_e4m3fn, True)
    path = os.path.join(tmp_path, "m.safetensors")
    save_file(full, path)
    modules, info = C.load_moe_layers(path, prefix=pre, device=dev)
    m = modules[layer]
    assert info["fp8_optimizations"] and m.experts[0].w1.weight.is_cuda and m.experts[0].w1.hdmoe_fp8_matrix_mult
    assert m._collect(x.to(dev).reshape(-1, 512)) is not None          # the one-call path applies
    from comfyui_amd import functional as HF
    y = m(x.to(dev))
    idx, w = HF.gate_top2(x.to(dev).reshape(-1, 512), m.gate.weight)
    check_layer(sd, x, "fp8", y.cpu(), idx.cpu(), w.cpu(), 4)


def test_packed_pointers_are_reused_only_while_nothing_changed(dev):
    """The module keeps the pointer structures of the previous call while every weight and scale is the same tensor
    at the same address. It must notice: a Parameter's storage swapped under it (`p.data = ...`), a scale_input
    changed in place (after ops.invalidate_scale_cache(), as for ops.scale_value), train/eval of fp8_ops Linears;
    and it must not keep a replaced weight alive."""
    import gc
    import weakref
    from comfyui_amd import ops
    dim = 256
    sd, x = small_layer(seed=5, dim=dim, tokens=90, weights="fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    xd = x.to(dev)
    base = m(xd).cpu()
    assert torch.equal(m(xd).cpu(), base) and m.__dict__.get("_packed") is not None
    idx, w, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])

    def oracle(state):
        return O.moe_forward(x, oracle_params(state, 4), "fp8mm", gate_result=(idx, w))
    # (a) storage swapped in place
    lin = m.experts[1].w3
    old = weakref.ref(lin.weight.data)
    lin.weight.data = sd["experts.0.w3.weight"].to(dev).clone()
    sd2 = dict(sd)
    sd2["experts.1.w3.weight"] = sd["experts.0.w3.weight"]
    got = m(xd).cpu()
    close(got, oracle(sd2), 1e-2)
    assert not torch.equal(got, base)
    gc.collect()
    assert old() is None, "the replaced weight is still referenced"
    # (b) a scale_input value changed in place: visible after the documented invalidation
    with torch.no_grad():
        for e in range(4):
            m.experts[e].w2.scale_input.data.fill_(0.5)
        m.shared_experts.w2.scale_input.data.fill_(0.5)
    ops.invalidate_scale_cache()
    sd3 = dict(sd2)
    for k in sd3:
        if k.endswith("w2.scale_input"):
            sd3[k] = torch.tensor(0.5)
    close(m(xd).cpu(), oracle(sd3), 1e-2)
    # (c) another device tensor for x's device is the same key; a CPU-resident Linear drops the cache
    m.experts[0].w1.to("cpu")
    assert torch.equal(m(xd).cpu(), m(xd).cpu()) and m.__dict__.get("_packed") is None
