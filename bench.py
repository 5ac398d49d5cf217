#!/usr/bin/env python3
"""Benchmark of the HiDream MoE SwiGLU feed-forward layer on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg2|cfg1|cfg5-256|cfg5-4096|cfg3-branch|cfg3-bf16|cfg4 [--layers L]] [--aux-kernels] [--no-cpu-baseline]

A step is one forward of comfyui_amd.hidream.MOEFeedForwardSwiGLU (gate, dispatch, quantise,
grouped fp8 GEMMs, combine, shared expert) over one synthetic batch that is already resident in
HBM. The default workload is the headline configuration: 8192 tokens (2 x 4096), fp8 e4m3fn
weights with per-tensor scales, activations N(0,1) with 1 % of the channels scaled by 20.

Order of a run: 40 untimed layer passes and the untimed per-stage passes (their count is reported as
`untimed_forwards_before_warmup`), then the W warm-up steps, then the K timed steps. The first 30 or so forwards
of a process run 5-25 % slower than the ones after them (code objects loading, then the clock settling under the
load), so a run whose W and K are small would otherwise time the start of the process instead of the layer.

Prints ONE JSON line. `value` is tokens/s over the K timed steps. `roofline` describes the
dominant kernel (the grouped gate/up GEMM with the SiLU*mul epilogue): its algorithmic FLOP per
launch divided by its average duration, measured with HIP events recorded on the launch stream
around that kernel inside the timed steps. `cpu_baseline` is the CPU oracle's restatement of the
reference's `--cpu` dataflow (fp32 compute, fp8 weights dequantised per call) timed on this
host's cores over a bounded sample of the same batch.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E



def gate_up_kernel_name(T, D, H, Hs, E, fp8=True):
    """Which kernel the library's launcher runs for the gate/up contraction of a layer: asked of the library itself
    (hdmoe_gate_up_kernel_name evaluates the launcher's rule under the current form switches)."""
    from comfyui_amd import _lib
    return _lib.lib.hdmoe_gate_up_kernel_name(_lib.W_E4M3FN if fp8 else _lib.W_BF16, T, E, D, H, Hs, 1).decode()


def measured_traffic(workload):
    """L2-side traffic of the dominant kernel per launch (bytes fetched + written) as the last rocprofv3 --pmc runs
    measured it: profiles/traffic.json holds, per workload, the calibrated FETCH_SIZE and WRITE_SIZE readings, the
    commit they were taken at and the summary file they come from. None for a workload that was not profiled."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            entry = json.load(f).get(workload)
    except (OSError, ValueError):
        return None, None
    if not entry:
        return None, None
    return entry["fetch_bytes"] + entry["write_bytes"], entry


class HipEvents:
    """hipEvent_t handles through the HIP runtime that torch already loaded; they can be recorded
    from inside the library on the stream the kernels are launched on."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def create(self, n):
        out = []
        for _ in range(n):
            e = ctypes.c_void_p()
            rc = self.hip.hipEventCreate(ctypes.byref(e))
            if rc != 0:
                raise RuntimeError(f"hipEventCreate failed: {rc}")
            out.append(e.value)
        return out

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        self.hip.hipEventSynchronize(b)
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return ms.value

    def destroy(self, evs):
        for e in evs:
            self.hip.hipEventDestroy(e)


def flops_per_token(D, H, Hs, E, K=2):
    gate_up = K * 2 * 2 * D * H + 2 * 2 * D * Hs
    down = K * 2 * D * H + 2 * D * Hs
    return dict(gate=2 * D * E, gate_up=gate_up, down=down, total=gate_up + down + 2 * D * E)


def cpu_baseline(cfg, sd, sample_tokens):
    """The oracle's restatement of the reference's --cpu path on a bounded sample."""
    from oracle import hidream_moe_oracle as O
    params = O.oracle_params(sd, 4)
    mode = "upcast" if cfg["weights"] == "fp8" else "plain"
    x2 = cfg["x"].reshape(-1, cfg["x"].shape[-1]).float()  # --cpu computes in fp32
    gate = params["gate"].float()
    params = dict(params, gate=gate)
    if mode == "plain":
        for ffn in params["experts"] + [params["shared"]]:
            for lp in ffn:
                lp.weight = lp.weight.float()   # --cpu upcasts bf16 checkpoints once at load
    xs = x2[:sample_tokens].unsqueeze(0).contiguous()
    O.moe_forward(x2[:32].unsqueeze(0).contiguous(), params, mode)  # warm caches / thread pool
    reps, dt = 0, 0.0
    t0 = time.perf_counter()
    while reps < 10 and dt < 10.0:   # about 10 s of CPU work, at most 10 forwards
        O.moe_forward(xs, params, mode)
        reps += 1
        dt = time.perf_counter() - t0
    return dict(value=reps * sample_tokens / dt, unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{reps} forward(s) over the first {sample_tokens} tokens of the same batch through the oracle's "
                       f"restatement of the reference --cpu dataflow (fp32 compute, mode={mode}, fp8 weights dequantised "
                       f"per call), {dt:.2f} s, torch CPU threads={torch.get_num_threads()}, os.cpu_count()={os.cpu_count()}")


def aux_kernels(dev, module, x):
    """Stand-alone timings of the kernels around the layer: algorithmic bytes / time against the HBM figure."""
    from comfyui_amd import functional as HF
    B, S, D = x.shape
    T = B * S
    g = torch.Generator().manual_seed(2)
    shift, scale, gate = ((torch.randn((B, D), generator=g) * 0.3).to(torch.bfloat16).to(dev) for _ in range(3))
    x2 = x.reshape(T, D)
    idx, w = HF.gate_top2(x2, module.gate.weight)
    _, _, perm, inv = HF.dispatch(idx, len(module.experts))
    y = torch.randn((2 * T, D), device=dev).to(torch.bfloat16)
    sh = torch.randn((T, D), device=dev).to(torch.bfloat16)
    wt = module.experts[0].w1
    w32 = torch.randn(wt.weight.shape, device=dev) * 0.02

    def timed(fn, nbytes, reps=50):
        for _ in range(5):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        return {"ms": ms, "bytes": nbytes, "GBps": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBPS}

    def hunyuan_block(dtype, tokens=8192, dim=2048, inner=8192, E=8):
        """The sibling model's MoE block (Hunyuan3D-2.1: width 2048, 8 GELU experts of hidden 8192, top-2, shared
        expert) at 2 x 4096 latent tokens, random weights; TFLOP/s over the 6 Linears a token goes through."""
        from comfyui_amd import hunyuan3d as H
        m = H.MoEBlock(dim, num_experts=E, moe_top_k=2, ff_inner_dim=inner, dtype=dtype, device=dev).eval()
        gg = torch.Generator(device=dev).manual_seed(3)
        with torch.no_grad():
            for prm in m.parameters():
                prm.copy_((torch.randn(prm.shape, generator=gg, device=dev) / (prm.shape[-1] ** 0.5 if prm.dim() > 1 else 5.0)).to(dtype))
            xh = torch.randn((2, tokens // 2, dim), generator=gg, device=dev).to(dtype)
            r = timed(lambda: m(xh), 0, reps=20)
        flop = tokens * 3 * 2 * 2 * dim * inner
        return {"ms": r["ms"], "tokens": tokens, "TFLOPs": flop / r["ms"] / 1e9, "frac_of_mfma_peak": flop / r["ms"] / 1e9 / PEAK_BF16_TFLOPS}

    def fp8_gemm_vs_vendor():
        """One plain fp8 Linear, out = bf16((a . w^T) * scale), through this library's kernel (hdmoe_linear: the K loop of
        the feed-forward kernels with the trivial epilogue) and through torch._scaled_mm (the vendor library) on the same
        operands: e4m3fn casts of N(0,1) values, the data the matrix cores' clock depends on. M x N x K."""
        rows = []
        gg = torch.Generator(device=dev).manual_seed(5)
        one = torch.ones((), dtype=torch.float32, device=dev)
        for M, N, K in ((16384, 16384, 2560), (16384, 13824, 2560), (16384, 2560, 6912), (16384, 16384, 16384)):
            a = torch.randn((M, K), generator=gg, device=dev).to(torch.float8_e4m3fn)
            w = torch.randn((N, K), generator=gg, device=dev).to(torch.float8_e4m3fn)
            flop = 2.0 * M * N * K
            ours = timed(lambda: HF.linear(a, w, one, one), 0, reps=10)
            entry = {"M": M, "N": N, "K": K, "hdmoe_linear_ms": ours["ms"], "hdmoe_linear_TFLOPs": flop / ours["ms"] / 1e9}
            try:
                theirs = timed(lambda: torch._scaled_mm(a, w.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16), 0, reps=10)
                entry.update({"scaled_mm_ms": theirs["ms"], "scaled_mm_TFLOPs": flop / theirs["ms"] / 1e9})
            except (RuntimeError, NotImplementedError) as e:
                entry["scaled_mm_error"] = str(e)[:200]
            rows.append(entry)
            del a, w
        return rows

    def mfma_ceiling():
        """The matrix cores alone: a loop of fp8 MFMAs on register operands (csrc/mfma_probe.hip), one block of 8 waves
        per CU as the GEMM kernels run, on zeros and on e4m3fn casts of N(0,1) values. Rate from events around the
        launch; the clock from the kernel's own cycle counter against the device's constant-rate counter."""
        path = os.path.join(ROOT, "comfyui_amd", "libhdmoe_probe.so")
        if not os.path.exists(path):
            return {"error": "libhdmoe_probe.so is not built (python -m comfyui_amd.build)"}
        probe = ctypes.CDLL(path)
        probe.hdmoe_probe_mfma_fp8.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                               ctypes.c_void_p, ctypes.c_void_p]
        blocks, iters, nacc = 256, 4000, probe.hdmoe_probe_accumulators()
        wall_khz = probe.hdmoe_probe_wall_clock_khz()
        ticks = torch.zeros(2, dtype=torch.int64, device=dev)
        sink = torch.zeros(1, dtype=torch.float32, device=dev)
        gg = torch.Generator(device=dev).manual_seed(6)
        data = {"zeros": torch.zeros(blocks * 512 * 64, dtype=torch.uint8, device=dev),
                "normal": torch.randn(blocks * 512 * 64, generator=gg, device=dev).to(torch.float8_e4m3fn).view(torch.uint8)}
        out = {}
        stream = torch.cuda.current_stream().cuda_stream
        for form, name, per in ((0, "32x32x64", 131072), (1, "16x16x128", 65536)):
            for kind, buf in data.items():
                run = lambda: probe.hdmoe_probe_mfma_fp8(form, buf.data_ptr(), blocks, iters, ticks.data_ptr(), sink.data_ptr(), stream)
                r = timed(run, 0, reps=10)
                flop = float(blocks) * 8 * iters * nacc * per
                t = ticks.cpu().tolist()
                entry = {"ms": r["ms"], "TFLOPs": flop / r["ms"] / 1e9, "frac_of_published_peak": flop / r["ms"] / 1e9 / PEAK_FP8_TFLOPS}
                if wall_khz > 0 and t[1] > 0:
                    # the first wave's cycle counter against the constant-rate counter over its own run: the clock
                    # the matrix cores sustained under this instruction on this data
                    entry["shader_clock_GHz"] = t[0] / t[1] * wall_khz / 1e6
                out[f"{name}_{kind}"] = entry
        return out

    return {
        "fp8_gemm_vs_vendor": fp8_gemm_vs_vendor(),
        "mfma_ceiling": mfma_ceiling(),
        "hunyuan3d_moe_block_bf16": hunyuan_block(torch.bfloat16),
        "hunyuan3d_moe_block_fp16": hunyuan_block(torch.float16),
        "ln_modulate": timed(lambda: HF.ln_modulate(x2, scale, shift, S), 2 * T * D * 2),
        "combine": timed(lambda: HF.combine(y, inv, w, sh), 4 * T * D * 2 + T * 12),
        "combine_gated_residual": timed(lambda: HF.combine_gated_residual(y, inv, w, sh, gate, x2, S), 5 * T * D * 2 + T * 12),
        "stochastic_round_e4m3fn": timed(lambda: HF.stochastic_round_e4m3fn(w32, wt.scale_weight, 1), w32.numel() * 5),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg5-256", "cfg5-4096", "cfg3-branch", "cfg3-bf16", "cfg4"])
    ap.add_argument("--layers", type=int, default=48, help="cfg4 only: number of stacked layers")
    ap.add_argument("--cpu-sample-tokens", type=int, default=8192)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--aux-kernels", action="store_true",
                    help="also time the stand-alone kernels outside the layer (LayerNorm+modulation, gated-residual "
                         "combine, stochastic rounding of one expert weight), the plain fp8 Linear against the vendor "
                         "library's on the feed-forward's shapes and the matrix cores' own rate, and report them under "
                         "\"aux\"")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one plain 256 MiB device copy, whose FETCH_SIZE/WRITE_SIZE readings calibrate the counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on exactly one GPU (one MI355X holds the whole layer; tokens are "
              "independent, so more GPUs would only replicate it). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(1)

    from comfyui_amd import synth
    from comfyui_amd._lib import STAGE_NAMES

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    branch = args.workload.endswith("-branch")   # the block's whole feed-forward branch: x + gate * layer(LN-mod(x))
    stack = args.workload == "cfg4"              # 48 independent fp8 layers, x <- x + layer(LayerNorm(x)), 32768 tokens
    if stack:
        # weights and tokens are drawn on the device (11.5 GB of fp8 weights; the CPU generator would take minutes)
        modules = []
        for layer in range(args.layers):
            master, _ = synth.make_weights(layer, device=dev)
            modules.append(synth.build_module(synth.to_state_dict(master, "fp8"), "fp8", dev))
            del master
        g = torch.Generator(device=dev).manual_seed(1000)
        x = torch.randn((2, 16384, synth.DIM), generator=g, device=dev).to(torch.bfloat16)
        cfg, sd, module = dict(weights="fp8", x=None), None, modules[0]
        args.no_cpu_baseline = True              # the CPU baseline is quoted on the headline workload
    else:
        cfg = synth.make_config(args.workload.replace("-branch", "").replace("-bf16", ""))
        if args.workload.endswith("-bf16"):      # the headline tokens and weights with the weights kept in bf16
            cfg["weights"] = "bf16"
            args.no_cpu_baseline = True
        sd = synth.to_state_dict(cfg["master"], cfg["weights"])
        cfg["master"] = None
        module = synth.build_module({k: v.to(dev) for k, v in sd.items()}, cfg["weights"], dev)
        modules = [module]
        x = cfg["x"].to(dev)
    B, S, D = x.shape
    T = B * S
    H, Hs, E = synth.H_ROUTED, synth.H_SHARED, synth.NUM_EXPERTS
    fl = flops_per_token(D, H, Hs, E)

    if args.pmc_calibration:
        # known traffic: 256 MiB read + 256 MiB written by one elementwise copy kernel
        src_cal = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst_cal = torch.empty_like(src_cal)
        dst_cal.copy_(src_cal)
        torch.cuda.synchronize()
        del src_cal, dst_cal

    n_layers = len(modules)
    if stack:
        zero = torch.zeros((B, 1, D), dtype=torch.bfloat16, device=dev)
        one = torch.ones((B, 1, D), dtype=torch.bfloat16, device=dev)

        def forward(stage_events=None):
            h = x
            for i, m in enumerate(modules):
                ev = None if stage_events is None else stage_events[i * (len(STAGE_NAMES) + 1):(i + 1) * (len(STAGE_NAMES) + 1)]
                h = m.forward_branch(h, zero, zero, one, stage_events=ev)
            return h
    elif branch:
        g = torch.Generator().manual_seed(1)
        shift, scale, gate_mlp = ((torch.randn((B, 1, D), generator=g) * 0.3).to(torch.bfloat16).to(dev) for _ in range(3))
        forward = lambda **kw: module.forward_branch(x, shift, scale, gate_mlp, **kw)
    else:
        forward = lambda **kw: module(x, **kw)

    hip = HipEvents()
    with torch.no_grad():
        # The per-stage figures first: untimed passes with all events recorded (the dominant kernel's own time comes
        # from the timed steps below). A process's first 30 or so forwards run 5-25 % slower than the ones after them
        # (code objects loading, then the clock settling under the load: 1.02-1.25 ms against 0.96 ms per step at
        # the headline workload), so 40 layer passes go first, and these passes in turn leave the device in the state of
        # a running model when the W warm-up steps and the K timed steps begin. The count of all forwards in front of
        # the warm-up is reported as `untimed_forwards_before_warmup`.
        n_ev = len(STAGE_NAMES) + 1
        settle_steps = max(1, 40 // n_layers)
        for _ in range(settle_steps):
            y = forward()
        torch.cuda.synchronize()
        stage_steps = max(1, min(args.steps, 20))
        stage_sets = [hip.create(n_ev * n_layers) for _ in range(stage_steps)]
        for k in range(stage_steps):
            y = forward(stage_events=stage_sets[k])
        torch.cuda.synchronize()
        # gate + dispatch (+ the bf16 path's row permutation) as one interval: an event recorded between two short
        # kernels costs about as much as the kernels themselves, so the sum of the three stage times overstates it
        g0, g1 = STAGE_NAMES.index("gate"), STAGE_NAMES.index("quant_permute") + 1
        gd_sets = []
        for _ in range(stage_steps):
            evs = [None] * (n_ev * n_layers)
            for l in range(n_layers):
                evs[l * n_ev + g0], evs[l * n_ev + g1] = hip.create(2)
            gd_sets.append(evs)
        for k in range(stage_steps):
            y = forward(stage_events=gd_sets[k])
        torch.cuda.synchronize()
        gd_ms = 0.0
        for evs in gd_sets:
            for l in range(n_layers):
                gd_ms += hip.elapsed_ms(evs[l * n_ev + g0], evs[l * n_ev + g1])
                hip.destroy([evs[l * n_ev + g0], evs[l * n_ev + g1]])
        gd_ms /= stage_steps * n_layers
        # The same interval with the tokens freshly written by the kernel in front of the layer, as they are inside a
        # model (the block's previous kernel leaves them in the memory-side cache); in the loops above every forward
        # re-reads the same 42 MB after 1.4 GB of other traffic, i.e. from HBM, cold.
        gd_warm_ms = None
        if not stack and not branch:
            x_src = x.clone()
            warm_sets = []
            for _ in range(stage_steps):
                evs = [None] * n_ev
                evs[g0], evs[g1] = hip.create(2)
                warm_sets.append(evs)
            for k in range(stage_steps):
                x.copy_(x_src)
                y = forward(stage_events=warm_sets[k])
            torch.cuda.synchronize()
            gd_warm_ms = 0.0
            for evs in warm_sets:
                gd_warm_ms += hip.elapsed_ms(evs[g0], evs[g1])
                hip.destroy([evs[g0], evs[g1]])
            gd_warm_ms /= stage_steps
            del x_src
        untimed_forwards = settle_steps + 2 * stage_steps + (stage_steps if gd_warm_ms is not None else 0)
        for _ in range(args.warmup):
            y = forward()
        torch.cuda.synchronize()
        # K timed steps. Inside them only the two events around the dominant kernel (the gate/up GEMM) are recorded
        # on the launch stream; recording all seven costs about 2 % of a step.
        dom = STAGE_NAMES.index("gemm_gate_up")
        ev_sets = []
        for _ in range(args.steps):
            evs = [None] * (n_ev * n_layers)
            for l in range(n_layers):
                evs[l * n_ev + dom], evs[l * n_ev + dom + 1] = hip.create(2)
            ev_sets.append(evs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(args.steps):
            y = forward(stage_events=ev_sets[k])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        dom_ms = 0.0
        for evs in ev_sets:
            for l in range(n_layers):
                dom_ms += hip.elapsed_ms(evs[l * n_ev + dom], evs[l * n_ev + dom + 1])
                hip.destroy([evs[l * n_ev + dom], evs[l * n_ev + dom + 1]])
        dom_ms /= args.steps * n_layers
    if bool(torch.isnan(y.float()).any()):
        print("bench.py: output contains NaN", file=sys.stderr)
        sys.exit(1)

    sec = (t1 - t0) / args.steps
    stage_ms = {n: 0.0 for n in STAGE_NAMES}
    for evs in stage_sets:
        for l in range(n_layers):
            base = l * (len(STAGE_NAMES) + 1)
            for i, n in enumerate(STAGE_NAMES):
                stage_ms[n] += hip.elapsed_ms(evs[base + i], evs[base + i + 1])
    for n in stage_ms:
        stage_ms[n] /= stage_steps * n_layers     # per layer
    stage_ms["gemm_gate_up"] = dom_ms             # from the timed steps
    for evs in stage_sets:
        hip.destroy(evs)

    fp8 = cfg["weights"] == "fp8"
    peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
    tokens_per_s = T / sec                        # through the whole stack when there is more than one layer
    tflops = tokens_per_s * n_layers * fl["total"] / 1e12
    gemm1_tflops = T * fl["gate_up"] / (stage_ms["gemm_gate_up"] * 1e-3) / 1e12
    gemm2_tflops = T * fl["down"] / (stage_ms["gemm_down"] * 1e-3) / 1e12
    eb = 1 if fp8 else 2
    gate_bytes = T * D * 2 + E * D * 2 + T * 2 * (4 + 2)
    # dispatch as built: index sort (the gate kernel counts, so the 2T ids are read once; write perm + inv_perm). fp8: the gate kernel also writes the
    # token's e4m3fn row, once, because every scale_input of these configurations is the same value (it would be three
    # rows, two routed slots + shared expert, with differing scales). Nothing is permuted for either weight type: the
    # gate/up GEMM reads the routed rows through the permutation.
    dispatch_bytes = (2 * T * 4) + 2 * (2 * T * 4) + (T * D if fp8 else 0)
    combine_bytes = 2 * T * D * 2 + T * D * 2 + T * D * 2 + T * 2 * 2 + 2 * T * 4

    traffic_bytes, traffic_entry = measured_traffic(args.workload)
    out = {
        "metric": "MoE-FFN tokens/sec at 8192 tok fp8" if args.workload == "cfg3" else f"MoE-FFN tokens/sec ({args.workload})",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "untimed_forwards_before_warmup": untimed_forwards,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8" if fp8 else "bf16",
        "data": "synthetic",
        "config": {
            "workload": {"cfg1": "cfg1: 1x1024 tokens, bf16 weights",
                         "cfg2": "cfg2: 1x4096 tokens, scaled fp8 e4m3fn weights, scale_input 1.0",
                         "cfg5-256": "cfg5: 256 tokens, fp8 weights, skewed routing (about 70% of tokens pick expert 0) "
                                     "with exact logit ties on every 64th token",
                         "cfg5-4096": "cfg5: 4096 tokens, fp8 weights, skewed routing (about 70% of tokens pick expert "
                                      "0) with exact logit ties on every 64th token",
                         "cfg4": f"cfg4: {n_layers} independent fp8 layers applied in sequence as x <- x + layer(LayerNorm(x)) "
                                 "(one enqueue per layer through forward_branch), 2x16384 = 32768 tokens; value counts "
                                 "tokens through the whole stack; stage_ms and roofline are per layer",
                         "cfg3-branch": "cfg3 tokens and weights through the block's whole feed-forward branch: x + gate_mlp * "
                                        "layer(LayerNorm(x) * (1 + scale_mlp) + shift_mlp), one enqueue (stage 'gate' "
                                        "includes the LayerNorm kernel, stage 'combine' the gated residual)",
                         "cfg3-bf16": "cfg3 tokens (2x4096 = 8192, 1% outlier channels x20) with bf16 weights",
                         "cfg3": "cfg3 (headline): 2x4096 = 8192 tokens x 2560, scaled fp8 e4m3fn weights "
                                 "(scale_weight = amax/448, scale_input = 1.0), bf16 gate, x ~ N(0,1) with 1% "
                                 "outlier channels x20, 4 routed experts (hidden 6912) top-2 + shared expert (hidden 3584)"}[args.workload],
            "tokens": T, "layers": n_layers, "dim": D, "hidden_routed": H, "hidden_shared": Hs, "experts": E, "top_k": 2,
        },
        "tflops": tflops,
        "pct_of_mfma_peak": 100.0 * tflops / peak,
        "flop_per_token": fl["total"],
        "gate_dispatch_GBps": (gate_bytes + dispatch_bytes) / (gd_ms * 1e-3) / 1e9,
        "gate_dispatch_bytes": gate_bytes + dispatch_bytes,
        "gate_dispatch_ms": gd_ms,
        "gate_dispatch_warm_ms": gd_warm_ms,
        "gate_dispatch_warm_GBps": None if gd_warm_ms is None else (gate_bytes + dispatch_bytes) / (gd_warm_ms * 1e-3) / 1e9,
        "combine_GBps": combine_bytes / (stage_ms["combine"] * 1e-3) / 1e9,
        "stage_ms": stage_ms,
        "gemm_down_tflops": gemm2_tflops,
        "roofline": {
            "kernel": gate_up_kernel_name(T, D, H, Hs, E, fp8=fp8),
            "bound": "mfma",
            "achieved": gemm1_tflops,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": gemm1_tflops / peak,
            "traffic": traffic_bytes,
            "traffic_note": ("rocprofv3 FETCH_SIZE + WRITE_SIZE per launch, calibrated against a plain copy; taken at commit "
                             f"{traffic_entry['commit']}, see profiles/{traffic_entry['source']}") if traffic_entry else None,
            "algorithmic_bytes": T * (3 * D * eb + (2 * H + Hs) * eb) + (E * 2 * H + 2 * Hs) * D * eb,
            "flop_per_launch": T * fl["gate_up"],
            "avg_launch_ms": stage_ms["gemm_gate_up"],
        },
    }
    if args.aux_kernels:
        out["aux"] = aux_kernels(dev, module, x)
        ceiling = out["aux"]["mfma_ceiling"].get("32x32x64_normal") if fp8 else None
        if ceiling:
            # the dominant kernel against what its own MFMA instruction sustains on this data on this device
            out["roofline"]["measured_ceiling_TFLOPs"] = ceiling["TFLOPs"]
            out["roofline"]["frac_of_measured_ceiling"] = gemm1_tflops / ceiling["TFLOPs"]
    if not args.no_cpu_baseline:
        del module
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline(cfg, sd, min(args.cpu_sample_tokens, T))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
