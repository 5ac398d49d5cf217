"""The two kernels of the fp8 gate/up contraction (8 waves: csrc/gemm.hip; 4 waves: csrc/swiglu4w.h; hdmoe_set_kernel_form
forces one or the other): same contraction and rounding points, so the same bytes out."""
import pytest
import torch

from comfyui_amd import synth
from oracle import hidream_moe_oracle as O
from tests.helpers import oracle_params, saved_forms, set_form, small_layer

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


@pytest.fixture
def four_wave():
    yield from saved_forms()


def grouped_swiglu(T, D, H, E, seed, dev, s_next):
    """h of hdmoe_grouped_swiglu on random routed rows, once per kernel form."""
    from comfyui_amd import _lib, functional as HF
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, D), generator=g).to(BF16)
    ws = []
    for _ in range(E):
        w1, s1 = synth.quantize_per_tensor(torch.randn((H, D), generator=g) * 0.03)
        w3, s3 = synth.quantize_per_tensor(torch.randn((H, D), generator=g) * 0.03)
        ws.append((w1.to(dev), s1.to(dev).float().reshape(()), w3.to(dev), s3.to(dev).float().reshape(())))
    if E >= 2:
        idx = torch.stack([torch.randperm(E, generator=g)[:2] for _ in range(T)]).to(torch.int32)
    else:
        idx = torch.zeros((T, 2), dtype=torch.int32)
    _, offsets, perm, _ = HF.dispatch(idx.to(dev), E)
    s_in = torch.tensor(1.0, device=dev)
    s_nx = torch.tensor(s_next, device=dev)
    xs = HF.quant_fp8(x.to(dev), s_in)[(perm // 2).long()].contiguous()

    def weights(w):
        f = _lib.FfnWeights()
        f.w1, f.w3, f.scale_w1, f.scale_w3 = w[0].data_ptr(), w[2].data_ptr(), w[1].data_ptr(), w[3].data_ptr()
        f.scale_in1 = f.scale_in3 = s_in.data_ptr()
        f.scale_in2 = s_nx.data_ptr()
        return f
    arr = (_lib.FfnWeights * E)(*[weights(w) for w in ws])
    out = []
    for form in ("0", "1"):
        set_form("HDMOE_SWIGLU4W", form)
        h = torch.full((2 * T, H), 0x55, dtype=torch.uint8, device=dev)
        _lib.check(_lib.lib.hdmoe_grouped_swiglu(_lib.W_E4M3FN, xs.data_ptr(), offsets.data_ptr(), 2 * T, E, D, H, arr,
                                                 h.data_ptr(), None))
        torch.cuda.synchronize()
        out.append(h.cpu())
    return out


@pytest.mark.parametrize("T,D,H,E,s_next", [
    (64, 2048, 128, 1, 1.0),        # one tile, the fewest K steps the kernel takes (16)
    (300, 2048, 256, 2, 0.5),       # partial tiles, a scale for the consuming Linear that is not 1
    (1500, 2560, 1024, 4, 0.37),    # one tile per block
    (5000, 2048, 3584, 3, 1.0),     # several tiles per block: the epilogue of one rides in the K loop of the next
    (777, 4096, 384, 5, 2.0),       # 16 pairs of K steps, an odd number of feature tiles
    (40, 2304, 256, 16, 1.0),       # 16 experts, most of them empty or a few rows; 9 pairs of K steps
    (3000, 6912, 256, 2, 0.25),     # the down projection's K as the contraction length (27 pairs)
])
def test_same_bytes_from_both_kernels(dev, four_wave, T, D, H, E, s_next):
    base, four = grouped_swiglu(T, D, H, E, seed=T + H, dev=dev, s_next=s_next)
    assert not bool((base == 0x55).all())
    assert torch.equal(base, four)


def test_layer_through_the_four_wave_kernel(dev, four_wave):
    """The whole layer (rows gathered through the dispatch permutation, shared expert in the same launch) against
    the oracle and against the 8-wave kernel."""
    dim = 2048
    sd, x = small_layer(seed=91, dim=dim, tokens=700, weights="fp8", scale_in=0.5)
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    set_form("HDMOE_SWIGLU4W", "0")
    base = m(x.to(dev)).cpu()
    set_form("HDMOE_SWIGLU4W", "1")
    four = m(x.to(dev)).cpu()
    assert torch.equal(base.view(torch.int16), four.view(torch.int16))
    idx, w, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    ref = O.moe_forward(x, oracle_params(sd, 4), "fp8mm", gate_result=(idx, w))
    d = O.error_metrics(four, ref)
    assert d["rel_rms"] <= 1e-2, d


def test_dense_feed_forward_through_both_kernels(dev, four_wave):
    """hdmoe_ffn_swiglu (the shared expert / text feed-forward on its own: one static group, no gather)."""
    from comfyui_amd import hidream, ops
    FP8 = torch.float8_e4m3fn
    dim, hidden = 2048, 1536
    g = torch.Generator().manual_seed(5)
    cls = ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=True, override_dtype=FP8)
    ff = hidream.FeedForwardSwiGLU(dim, hidden, dtype=BF16, device=dev, operations=cls).eval()
    for lin in (ff.w1, ff.w2, ff.w3):
        w8, sw = synth.quantize_per_tensor(torch.randn(tuple(lin.weight.shape), generator=g) * 0.03)
        lin.weight = torch.nn.Parameter(w8.to(dev), requires_grad=False)
        with torch.no_grad():
            lin.scale_weight.copy_(sw)
            lin.scale_input.fill_(0.5)
    x = torch.randn((2, 450, dim), generator=g).to(BF16).to(dev)
    set_form("HDMOE_SWIGLU4W", "0")
    base = ff(x).cpu()
    set_form("HDMOE_SWIGLU4W", "1")
    four = ff(x).cpu()
    assert bool(torch.isfinite(base.float()).all()) and float(base.float().abs().max()) > 0
    assert torch.equal(base.view(torch.int16), four.view(torch.int16))


def test_layer_with_the_four_wave_kernel_in_a_graph(dev, four_wave):
    """Capture and replay of a layer whose gate/up contraction takes the 4-wave kernel (no memset nodes, nothing
    allocated, the kernel attribute set before the capture)."""
    set_form("HDMOE_SWIGLU4W", "1")
    dim = 2048
    sd, x = small_layer(seed=17, dim=dim, tokens=600, weights="fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim)
    xs = [x.to(dev), (x * 0.5).to(dev), x.flip(1).contiguous().to(dev)]
    eager = [m(v).clone() for v in xs]
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


def test_random_shapes_same_bytes(dev, four_wave):
    """A seeded walk over token counts, widths, expert counts and cast scales."""
    import random
    rnd = random.Random(7)
    for it in range(12):
        E = rnd.choice([1, 2, 3, 4, 6, 8])
        D = rnd.choice([2048, 2304, 2560, 3072, 4096])
        H = 128 * rnd.randint(1, 12)
        T = rnd.choice([1, 7, 33, 100, 257, 511, 1000, 2049])
        s_next = rnd.choice([1.0, 0.5, 0.37, 2.0])
        base, four = grouped_swiglu(T, D, H, E, seed=500 + it, dev=dev, s_next=s_next)
        assert torch.equal(base, four), (T, D, H, E, s_next)
