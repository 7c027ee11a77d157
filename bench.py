"""Benchmark of the scattered-MoE layer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tokens N] [--no-cpu-baseline]

A step is one forward of the MoE layer (router -> sort/bin -> up-projection + SwiGLU -> down-projection
-> combine) over one batch of seeded synthetic tokens that already sit in HBM.  The default workload is
the Granite-3B-A800M-shape layer (32768 tokens, hidden 1536, 40 experts, top-8, intermediate 512, bf16,
Zipf(1.1) expert load).  One JSON line is printed:

* ``value``         tokens/s of the whole forward, K steps between two device synchronisations
* ``roofline``      the dominant kernel (grouped up-projection GEMM with fused SwiGLU; for the decode
                    workload the fp8 up-projection weight stream): algorithmic flops (or bytes) per
                    launch / average launch duration, measured with HIP events on the launch stream
                    in a second, instrumented run of the same K steps
* ``cpu_baseline``  the eager per-expert-loop path (the oracle, a port of the reference's eager
                    branch) in fp32 on the host cores, on a bounded token sample of the same workload
* ``workloads``     (default run only) the other four parity configurations, measured the same way in a few
                    seconds each: ms per step, the dominant kernel's roofline fraction, both grouped GEMMs
                    together, and the whole layer's algorithmic bytes over HBM peak (the decode target); the
                    decode workload also with the latency of ONE forward (launch, synchronise; median) and of
                    one replay of the forward captured in a HIP graph
* ``ceilings``      (default run only) what this GPU does, in this process, on work of the same size with no
                    gather, no expert boundaries and no activation: the vendor library's dense bf16 GEMM
                    (torch.mm) of both grouped GEMMs' shapes on the same random data, and a 1 GiB copy
* ``training``      (default run, or --backward) one training step of the layer (forward + backward for x and
                    every parameter) through the kernel branch and through the eager branch, with the stage
                    times of the kernel branch and the weight-gradient kernel's rate
* ``block_fusion``  (default run only) the two fusions with the transformer block around the layer, each against
                    the separate calls: RMSNorm + router, and combine + shared-expert sum + residual tail
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP32_TFLOPS = 157.3   # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

def measured_traffic(workload):
    """HBM-side bytes per launch of the dominant kernel, from the committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    summary of this workload (profiles/moe_layer_<workload>.txt: its header gives the commands and the calibration
    against a 256 MiB copy, its traffic table ends in a line `dominant kernel HBM traffic per launch (bytes): N`).
    A counter cannot be read from inside this process, so the figure is taken from that file; None without it."""
    path = os.path.join(ROOT, "profiles", f"moe_layer_{workload}.txt")
    key = "dominant kernel HBM traffic per launch (bytes):"
    try:
        for line in open(path):
            if line.startswith(key):
                return float(line[len(key):].split()[0]), os.path.relpath(path, ROOT)
    except (OSError, ValueError, IndexError):
        pass
    return None, None


class StageTimer:
    """HIP events (torch.cuda.Event on the current stream, which is the stream the kernels are
    launched on) around every stage of the forward."""

    def __init__(self):
        import torch

        self.torch = torch
        self.events = {}
        self._open = {}

    def begin(self, name):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self._open[name] = ev

    def end(self, name):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self.events.setdefault(name, []).append((self._open.pop(name), ev))

    def summary(self):
        self.torch.cuda.synchronize()
        return {n: sum(a.elapsed_time(b) for a, b in evs) / len(evs) for n, evs in self.events.items()}

    def per_step(self, steps):
        """Total time of every stage per step (a stage may run several times in one step)."""
        self.torch.cuda.synchronize()
        return {n: sum(a.elapsed_time(b) for a, b in evs) / steps for n, evs in self.events.items()}


def build_module(w, inputs, device, fp8_tiled=True):
    import torch

    from dolomite_engine_amd import MoE

    with torch.device("meta"):
        m = MoE(hidden_size=w.H, intermediate_size=w.I, shared_intermediate_size=None, num_experts=w.E,
                num_experts_per_tok=w.k, activation_function="swiglu", add_bias=False, dropout=0.0,
                init_method="normal", initializer_range=0.02, m_width=None, num_layers=1,
                use_padding_free_transformer=True)
    m = m.to(w.dtype).to_empty(device=device).eval()
    with torch.no_grad():
        m.gate.weight.copy_(inputs["gate_w"])
        if w.fp8:
            m.c_fc.set_fp8_weight(inputs["w_fc"].to(device), inputs["fc_scale"].to(device), w.dtype,
                                  tiled=fp8_tiled, glu=True)
            m.c_proj.set_fp8_weight(inputs["w_proj"].to(device), inputs["proj_scale"].to(device), w.dtype,
                                    tiled=fp8_tiled, glu=False)
        else:
            m.c_fc.weight.copy_(inputs["w_fc"])
            m.c_proj.weight.copy_(inputs["w_proj"])
    if inputs["bias"] is not None:
        m.router_logit_bias = inputs["bias"].to(device)
    return m


METRIC = "MoE fwd tokens/s & % bf16 MFMA peak, Granite-3B-A800M layer, 1 GPU"  # the headline metric string, for the default workload


def metric_name(w):
    if w.name == "granite-3b-a800m":
        return METRIC
    what = "% HBM peak" if w.fp8 else ("% fp32 MFMA peak" if w.dtype == __import__("torch").float32 else "% bf16 MFMA peak")
    return f"MoE fwd tokens/s & {what}, {w.name} layer, 1 GPU"


def layer_algorithmic_bytes(w, touched):
    """Compulsory HBM traffic of one forward: x once, every touched expert's weights (and fp8 scales) once, the
    gate weight, y once, and the routing metadata (sorted order: two int32 per slot, gates, offsets)."""
    elt = 2 if w.dtype != __import__("torch").float32 else 4
    welt = 1 if w.fp8 else elt
    L = w.T * w.k
    weights = touched * (3 * w.I * w.H) * welt + (touched * (2 * w.I + w.H) * 4 if w.fp8 else 0)
    return w.T * w.H * elt * 2 + weights + w.E * w.H * elt + L * (4 + 4 + elt) + 4 * w.E


def measure_compact(name, device, steps=20, warmup=5):
    """One of the other workloads, timed like the headline: K forwards between two synchronisations, then an
    instrumented run with HIP events around every stage."""
    import torch

    from dolomite_engine_amd import Kernel, enable_kernels, ops
    from oracle import moe_oracle as oracle

    w = oracle.WORKLOADS[name]
    inputs = oracle.make_inputs(w)
    m = build_module(w, inputs, device)
    x = inputs["x"].to(device)
    L = w.T * w.k
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        for _ in range(warmup):
            m(x)
        torch.cuda.synchronize()
        # The GPU has been idle (CPU baseline, set-up of this workload) and a 0.1 - 0.5 ms step does not bring its
        # clocks back up within five steps: warm up for at least 50 ms and time at least 30 ms.
        t0 = time.perf_counter()
        m(x)
        torch.cuda.synchronize()
        est = max(time.perf_counter() - t0, 1e-5)
        for _ in range(int(0.05 / est) + 1):
            m(x)
        torch.cuda.synchronize()
        steps = max(steps, int(0.03 / est) + 1)
        t0 = time.perf_counter()
        for _ in range(steps):
            m(x)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        timer = StageTimer()
        ops.set_stage_timer(timer)
        for _ in range(steps):
            m(x)
        stages = timer.summary()
        ops.set_stage_timer(None)
        _, _, idx = m._compute_routing_weights(x)
        touched = int((torch.bincount(idx.flatten().long(), minlength=w.E) > 0).sum())
    out = {"ms_per_step": ms, "tokens_per_s": w.T / (ms * 1e-3), "dtype": str(w.dtype).replace("torch.", ""),
           "layer_tflops": 6.0 * L * w.H * w.I / (ms * 1e-3) / 1e12, "stages_ms": stages}
    layer_bytes = layer_algorithmic_bytes(w, touched)
    out["layer_hbm_frac"] = layer_bytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS
    if w.fp8:
        up_bytes = touched * (2 * w.I * w.H) + touched * 2 * w.I * 4 + w.T * w.H * 2 + L * w.I * 2 + L * 4 + w.E * 4
        out["kernel"], out["bound"] = "up_swiglu_fp8", "hbm"
        out["frac"] = up_bytes / (stages["up_swiglu_fp8"] * 1e-3) / 1e9 / PEAK_HBM_GBS
        out.update(measure_latency(m, x))
    else:
        peak = PEAK_FP32_TFLOPS if w.dtype == torch.float32 else PEAK_BF16_TFLOPS
        out["kernel"], out["bound"] = "up_swiglu", "mfma"
        out["frac"] = 4.0 * L * w.H * w.I / (stages["up_swiglu"] * 1e-3) / 1e12 / peak
        out["both_gemms_frac"] = (6.0 * L * w.H * w.I / ((stages["up_swiglu"] + stages["scattered_gemm"]) * 1e-3)
                                  / 1e12 / peak)
    del m, x, inputs
    torch.cuda.empty_cache()
    return out


def _time_ms(fn, iters, warmup=3):
    """Average duration of ``fn()`` over ``iters`` launches between two HIP events on the current stream."""
    import torch

    for _ in range(warmup):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def measure_ceilings(w, inputs, device, iters=20):
    """What the same GPU does in the same process on the same amount of work without the layer's structure:
    the vendor library's dense GEMM (torch.mm, bf16) for both grouped GEMMs' shapes -- L rows of N(0,1) data against
    ONE expert's N(0,0.02) weights, no gather, no expert boundaries, no SwiGLU, contiguous output -- and a 1 GiB
    device-to-device copy.  The grouped kernels cannot be expected to beat these; the distance to them is what the
    gather, the expert tails and the epilogue cost."""
    import torch

    L = w.T * w.k
    g = torch.Generator(device="cpu").manual_seed(99)
    out = {}
    w_fc = inputs["w_fc"][0].to(device)          # (2I, H)
    w_proj = inputs["w_proj"][0].to(device)      # (H, I)
    xs = torch.randn(1024, w.H, generator=g).to(w.dtype).to(device).repeat(L // 1024 + 1, 1)[:L].contiguous()
    # (rows repeat every 1024: the data stays random for the multipliers, and drawing 400 M normals on the host
    #  would take longer than everything else in this file)
    xs += torch.arange(L, device=device, dtype=torch.float32).mul_(1e-6).to(w.dtype).unsqueeze(1)
    acts = torch.randn(1024, w.I, generator=g).mul_(0.3).to(w.dtype).to(device).repeat(L // 1024 + 1, 1)[:L].contiguous()
    up_out = torch.empty((L, 2 * w.I), dtype=w.dtype, device=device)
    down_out = torch.empty((L, w.H), dtype=w.dtype, device=device)
    peak = PEAK_BF16_TFLOPS
    ms = _time_ms(lambda: torch.mm(xs, w_fc.t(), out=up_out), iters)
    fl = 2.0 * L * w.H * 2 * w.I
    out["dense_up_gemm"] = {"shape": f"({L} x {w.H}) @ ({2 * w.I} x {w.H})^T", "ms": ms,
                            "tflops": fl / (ms * 1e-3) / 1e12, "frac": fl / (ms * 1e-3) / 1e12 / peak}
    ms2 = _time_ms(lambda: torch.mm(acts, w_proj.t(), out=down_out), iters)
    fl2 = 2.0 * L * w.I * w.H
    out["dense_down_gemm"] = {"shape": f"({L} x {w.I}) @ ({w.H} x {w.I})^T", "ms": ms2,
                              "tflops": fl2 / (ms2 * 1e-3) / 1e12, "frac": fl2 / (ms2 * 1e-3) / 1e12 / peak}
    out["dense_both_gemms_frac"] = (fl + fl2) / ((ms + ms2) * 1e-3) / 1e12 / peak
    del xs, acts, up_out, down_out
    src = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_(0, 255)
    dst = torch.empty_like(src)
    ms3 = _time_ms(lambda: dst.copy_(src), 10)
    out["copy_1gib"] = {"ms": ms3, "gbs_read_plus_write": 2.0 * (1 << 30) / (ms3 * 1e-3) / 1e9,
                        "frac": 2.0 * (1 << 30) / (ms3 * 1e-3) / 1e9 / PEAK_HBM_GBS}
    del src, dst
    out["gemm_inner_loop"] = measure_inner_loop_probes(device)
    out["note"] = ("torch.mm (vendor dense bf16 GEMM) and Tensor.copy_ timed with HIP events in this process; "
                   "gemm_inner_loop: the library's diagnostic kernels (mi_moe_probe_kloop) on random bf16 data; "
                   "frac is of the 2.5 PFLOP/s bf16 MFMA peak / the 8 TB/s HBM peak")
    torch.cuda.empty_cache()
    return out


def measure_inner_loop_probes(device, slices=6144):
    """The pieces of the persistent grouped GEMM's inner loop in isolation (mi_moe_probe_kloop: one workgroup per
    CU, the GEMM's own 256 x 256 tile, slice, ring and schedule, on 2 MiB of L2-resident random bf16 data): the
    matrix instructions alone, with the LDS fragment reads, the L2 -> LDS DMA alone, and all of it together.  What
    "all of it" reaches is the ceiling of the GEMM's K loop on this GPU -- before gather, expert tails, tile
    boundaries and epilogues."""
    import torch

    from dolomite_engine_amd import _lib

    lib = _lib.load()
    g = torch.Generator(device="cpu").manual_seed(7)
    data = torch.randn((2 << 20) // 2 + 4096, generator=g).to(torch.bfloat16).to(device)
    sink = torch.empty(lib.mi_moe_probe_sink_bytes(), dtype=torch.uint8, device=device)
    cus = sink.numel() // (512 * 4)
    stream = torch.cuda.current_stream().cuda_stream
    out = {"workgroups": cus, "slices_per_workgroup": slices}
    for mode, name in ((0, "mfma_only"), (1, "mfma_plus_lds_reads"), (2, "dma_only"), (3, "all_pingpong")):
        def launch():
            _lib.check(lib.mi_moe_probe_kloop(mode, data.data_ptr(), data.numel() * 2, slices, sink.data_ptr(),
                                              sink.numel(), stream))
        ms = _time_ms(launch, 5, warmup=2)
        rec = {"ms": ms}
        if mode != 2:
            tf = 2.0 * 256 * 256 * 32 * slices * cus / (ms * 1e-3) / 1e12
            rec.update(tflops=tf, frac=tf / PEAK_BF16_TFLOPS)
        if mode >= 2:
            rec["l2_to_lds_tbs"] = 32768.0 * slices * cus / (ms * 1e-3) / 1e12
        out[name] = rec
    del data, sink
    return out


def measure_training(m, x, w, steps, full=False):
    """One training step of the layer (forward + backward for the input and every parameter, a synthetic upstream
    gradient, the auxiliary loss included) through the kernel branch and through the eager branch."""
    import torch

    from dolomite_engine_amd import Kernel, enable_kernels, ops
    from dolomite_engine_amd.loss import clear_aux_loss, get_aux_loss

    m.train()
    xg = x.clone().requires_grad_(True)
    dy = torch.randn_like(x)

    def train_step(kernels: bool):
        m.zero_grad(set_to_none=True)
        xg.grad = None
        clear_aux_loss()
        if kernels:
            with enable_kernels([Kernel.scattermoe]):
                out_ = m(xg)
        else:
            out_ = m(xg)
        # the upstream gradient goes straight into autograd: no loss kernels of the bench's own in the step
        aux = get_aux_loss()
        if torch.is_tensor(aux) and aux.requires_grad:
            torch.autograd.backward([out_, aux], [dy, torch.full_like(aux, 0.01)])
        else:
            out_.backward(dy)

    train = {}
    # kernels: the up-projection's pre-activation is kept for the backward (the module's default);
    # kernels_recompute: it is recomputed there (MoE.keep_preactivation = False)
    variants = [("kernels", True), ("eager", False)]
    if full:
        variants.insert(1, ("kernels_recompute", True))
    for name, kernels in variants:
        m.keep_preactivation = name != "kernels_recompute"
        torch.cuda.reset_peak_memory_stats()
        for _ in range(3):
            train_step(kernels)
        torch.cuda.synchronize()
        train["peak_mem_gib_" + name] = torch.cuda.max_memory_allocated() / 2 ** 30
        n = max(3, steps // 5)
        t0 = time.perf_counter()
        for _ in range(n):
            train_step(kernels)
        torch.cuda.synchronize()
        train["ms_per_step_fwd_bwd_" + name] = (time.perf_counter() - t0) / n * 1e3
    m.keep_preactivation = True
    timer = StageTimer()
    ops.set_stage_timer(timer)
    for _ in range(5):
        train_step(True)
    stages = timer.per_step(5)
    ops.set_stage_timer(None)
    train["stages_ms_fwd_bwd"] = stages
    train["kernel_stages_ms_sum"] = sum(stages.values())
    if "grouped_wgrad" in stages:
        # both weight gradients: d_w_fc 2 * L * 2I * H flops, d_w_proj 2 * L * H * I
        fl = 6.0 * w.T * w.k * w.H * w.I
        train["wgrad_tflops"] = fl / (stages["grouped_wgrad"] * 1e-3) / 1e12
        train["wgrad_frac"] = train["wgrad_tflops"] / PEAK_BF16_TFLOPS
    m.eval()
    m.zero_grad(set_to_none=True)
    del xg, dy
    torch.cuda.empty_cache()
    return train


def measure_block_fusion(m, x, w, iters=30):
    """The two fusions with the transformer block around the layer (ln_2 in front, shared-expert sum / m_residual /
    residual add behind), each against the separate calls it replaces."""
    import torch
    import torch.nn.functional as F

    from dolomite_engine_amd import ops

    out = {}
    with torch.no_grad():
        gamma = torch.ones(w.H, dtype=w.dtype, device=x.device)
        bias = m.router_logit_bias
        if ops.rmsnorm_router_fused_supported(x, w.E, w.k):
            def unfused():
                xn = F.rms_norm(x, (w.H,), gamma, 1e-5)
                return ops.router_fused(xn, m.gate.weight, w.k, bias=bias)

            out["rmsnorm_plus_router_ms"] = _time_ms(unfused, iters)
            out["rmsnorm_router_fused_ms"] = _time_ms(
                lambda: ops.rmsnorm_router_fused(x, gamma, 1e-5, m.gate.weight, w.k, bias=bias), iters)
        L = w.T * w.k
        o = torch.randn(1024, w.H, device=x.device).to(w.dtype).repeat(L // 1024, 1)
        gates = torch.rand(w.T, w.k, device=x.device).to(w.dtype)
        shared = torch.randn_like(x)
        residual = torch.randn_like(x)
        out["combine_ms"] = _time_ms(lambda: ops.combine(o, gates), iters)
        out["combine_then_shared_scale_residual_ms"] = _time_ms(
            lambda: (ops.combine(o, gates) + shared) * 0.22 + residual, iters)
        out["combine_block_tail_fused_ms"] = _time_ms(lambda: ops.combine(o, gates, shared, residual, 0.22), iters)
        del o, gates, shared, residual
    torch.cuda.empty_cache()
    return out


def measure_latency(m, x, reps=300):
    """One forward at a time: launch, wait for the device, repeat; the median.  And the same forward captured into
    a HIP graph, one replay at a time."""
    import torch

    from dolomite_engine_amd import Kernel, enable_kernels

    out = {}
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        for _ in range(20):
            y = m(x)
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            y = m(x)
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        out["latency_ms"] = sorted(ts)[len(ts) // 2] * 1e3
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            m(x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = m(x)
        for _ in range(20):
            graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(y_static, y):
            raise RuntimeError("graph replay differs from the eager forward")
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        out["graph_replay_latency_ms"] = sorted(ts)[len(ts) // 2] * 1e3
        t0 = time.perf_counter()
        for _ in range(reps):
            graph.replay()
        torch.cuda.synchronize()
        out["graph_replay_ms"] = (time.perf_counter() - t0) / reps * 1e3
        del graph, y_static
    return out


def measure_routing_stage(device, iters=30):
    """The routing stage by itself at the workloads' shapes and at shapes with more experts: router (gate GEMM +
    top-k + softmax), router + sort as the layer calls them, the stand-alone top-k + softmax on given logits, and
    torch's linear + topk (no softmax, no sort) on the same inputs.  HIP events around back-to-back calls;
    ``hbm_frac`` is the router's algorithmic bytes (x once, gate weights once, gates and indices out) over its time,
    against the HBM peak."""
    import torch
    import torch.nn.functional as F

    from dolomite_engine_amd import ops

    shapes = [  # tokens, hidden, experts, k, dtype
        (64, 4096, 64, 6, torch.bfloat16), (2048, 1536, 40, 8, torch.bfloat16), (16384, 1024, 32, 8, torch.bfloat16),
        (32768, 1536, 40, 8, torch.bfloat16), (131072, 1536, 40, 8, torch.bfloat16),
        (16384, 4096, 64, 6, torch.bfloat16), (64, 4096, 128, 8, torch.bfloat16), (64, 7168, 256, 8, torch.bfloat16),
        (4096, 2048, 128, 8, torch.bfloat16),
        (32768, 2048, 128, 8, torch.bfloat16), (8192, 7168, 256, 8, torch.bfloat16),
        (512, 256, 8, 2, torch.float32), (32768, 1536, 40, 8, torch.float32),
    ]
    g = torch.Generator(device="cpu").manual_seed(7)
    rows = []
    for T, H, E, k, dtype in shapes:
        x = torch.randn(T, H, generator=g).to(dtype).to(device)
        gw = (torch.randn(E, H, generator=g) * 0.02).to(dtype).to(device)
        elt = x.element_size()
        logits = F.linear(x, gw)
        row = {"tokens": T, "hidden": H, "experts": E, "top_k": k, "dtype": str(dtype).replace("torch.", "")}
        ms = _time_ms(lambda: ops.router_fused(x, gw, k), iters)
        nbytes = T * H * elt + E * H * elt + T * k * (elt + 4)
        row["router_us"] = ms * 1e3
        row["router_hbm_frac"] = nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS
        if ops.router_fused_sort_supported(x, E, k):
            row["router_plus_sort_us"] = _time_ms(lambda: ops.router_fused_sort(x, gw, k), iters) * 1e3
        else:
            row["router_plus_sort_us"] = _time_ms(lambda: ops.sort_bin(ops.router_fused(x, gw, k)[2], E), iters) * 1e3
        row["topk_softmax_us"] = _time_ms(lambda: ops.router_topk_softmax(logits, k), iters) * 1e3
        row["torch_linear_topk_us"] = _time_ms(lambda: torch.topk(F.linear(x, gw), k), iters) * 1e3
        rows.append(row)
        del x, gw, logits
    return rows


def cpu_baseline(w, inputs, sample_tokens, budget_s=10.0):
    """Eager path of the oracle in fp32 on the host, on the first ``sample_tokens`` tokens: one warm-up, then as
    many timed forwards as fit ``budget_s`` seconds (2 to 8), median."""
    import torch

    from oracle import moe_oracle as oracle

    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    x = inputs["x"][:sample_tokens].float()
    gate_w = inputs["gate_w"].float()
    if w.fp8:
        w_fc = oracle.dequant_fp8(inputs["w_fc"], inputs["fc_scale"])
        w_proj = oracle.dequant_fp8(inputs["w_proj"], inputs["proj_scale"])
    else:
        w_fc, w_proj = inputs["w_fc"].float(), inputs["w_proj"].float()
    bias = inputs["bias"]

    def run():
        _, gates, idx = oracle.route(x, gate_w, w.k, bias=bias)
        return oracle.experts_eager(x, gates, idx, w_fc, w_proj)

    t0 = time.perf_counter()
    run()
    iters = max(2, min(8, int(budget_s / max(time.perf_counter() - t0, 1e-3))))
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    out = {
        "value": sample_tokens / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"first {sample_tokens} tokens of the workload, fp32 eager per-expert loop, 1 warm-up + {iters} "
                  f"timed forwards, median {med * 1e3:.1f} ms; host has {os.cpu_count()} logical cpus",
    }
    if not w.fp8 and w.dtype == torch.bfloat16:
        # the same loop in the model dtype (host bf16 GEMMs are often slower than fp32): one warm-up, one timed
        xb, gb, fb, pb = x.bfloat16(), gate_w.bfloat16(), w_fc.bfloat16(), w_proj.bfloat16()

        def run_bf16():
            _, gates, idx = oracle.route(xb, gb, w.k, bias=bias)
            return oracle.experts_eager(xb, gates, idx, fb, pb)

        run_bf16()
        t0 = time.perf_counter()
        run_bf16()
        out["value_model_dtype"] = sample_tokens / (time.perf_counter() - t0)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=40)  # ~50 ms: the clocks have settled (10 steps: 1 % slower)
    ap.add_argument("--workload", default="granite-3b-a800m")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--tokens", type=int, default=None,
                    help="run the workload's shape at another token count (same weights and routing bias; the "
                         "extra blocks of the default run are left out and the metric string says so)")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default workload only: skip the compact measurements of the other four configurations")
    ap.add_argument("--cpu-sample-tokens", type=int, default=None)
    ap.add_argument("--graph", action="store_true",
                    help="also capture the forward into a HIP graph and report the time of a replay "
                         "(ms_per_step_graph_replay); value / ms_per_step stay the eager module call")
    ap.add_argument("--fp8-row-major", action="store_true",
                    help="decode workload: keep the fp8 expert weights row-major instead of in the streamed-tile layout")
    ap.add_argument("--backward", action="store_true",
                    help="also time a training step of the layer (forward + backward for the input and every "
                         "parameter, synthetic upstream gradient) through the kernel branch and through the eager "
                         "branch; reported as extra fields, value / ms_per_step stay the forward")
    ap.add_argument("--routing", action="store_true",
                    help="measure the routing stage alone (router, router + sort, top-k) at a list of shapes, "
                         "print them as one JSON line and exit")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one 256 MiB device-to-device copy so that a rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE run of this command contains a kernel of known traffic to scale by")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (one GPU's share of the layer at its real shape); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from dolomite_engine_amd import Kernel, enable_kernels, ops
    from oracle import moe_oracle as oracle

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.routing:
        print(json.dumps({"routing_stage": measure_routing_stage(device), "unit": "us per call, HIP events",
                          "peak_hbm_gbs": PEAK_HBM_GBS}))
        return

    w = oracle.WORKLOADS[args.workload]
    if args.tokens is not None:
        import dataclasses

        if args.tokens < 1:
            print("bench.py: --tokens must be positive", file=sys.stderr)
            sys.exit(2)
        w = dataclasses.replace(w, T=args.tokens)
    inputs = oracle.make_inputs(w)
    m = build_module(w, inputs, device, fp8_tiled=not args.fp8_row_major)
    x = inputs["x"].to(device)
    T, H, E, k, I = w.T, w.H, w.E, w.k, w.I
    L = T * k

    if args.pmc_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        for _ in range(args.warmup):
            y = m(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = m(x)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0

        graph_ms = None
        if args.graph:
            # the same forward captured once into a HIP graph and replayed: what a serving loop would run
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                m(x)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                y_static = m(x)
            for _ in range(args.warmup):
                graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms = (time.perf_counter() - t0) / args.steps * 1e3
            if not torch.equal(y_static, y):
                print("bench.py: graph replay differs from the eager forward", file=sys.stderr)
                sys.exit(1)

        # instrumented run of the same steps: HIP events around every stage
        timer = StageTimer()
        ops.set_stage_timer(timer)
        for _ in range(args.steps):
            y = m(x)
        stages = timer.summary()
        ops.set_stage_timer(None)

        idx = m._compute_routing_weights(x)[2]
        counts = torch.bincount(idx.flatten().long(), minlength=E).cpu()

    if args.backward and w.fp8:
        print("bench.py: --backward needs a 16-bit workload", file=sys.stderr)
        sys.exit(2)

    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = T / (elapsed / args.steps)
    flops = 6.0 * L * H * I
    touched = int((counts > 0).sum())

    # (the committed profiles are of the workloads' own token counts)
    traffic, traffic_src = measured_traffic(w.name) if args.tokens is None else (None, None)
    if w.fp8 and "up_swiglu_fp8" not in stages:
        roofline = None  # a batch so large that the weights were widened for the call: see stages_ms
    elif w.fp8:
        up_name = "up_swiglu_fp8"
        up_bytes = touched * (2 * I * H) + touched * 2 * I * 4 + T * H * 2 + L * I * 2 + L * 4 + E * 4
        ach = up_bytes / (stages[up_name] * 1e-3) / 1e9
        roofline = {"kernel": up_name, "bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": ach / PEAK_HBM_GBS, "traffic": traffic, "traffic_source": traffic_src,
                    "algorithmic_bytes": up_bytes,
                    "avg_launch_ms": stages[up_name]}
    else:
        up_name = "up_swiglu"
        up_flops = 4.0 * L * H * I
        peak = PEAK_FP32_TFLOPS if w.dtype == torch.float32 else PEAK_BF16_TFLOPS
        ach = up_flops / (stages[up_name] * 1e-3) / 1e12
        roofline = {"kernel": up_name, "bound": "mfma", "achieved": ach, "peak": peak,
                    "unit": "TFLOP/s", "frac": ach / peak, "traffic": traffic, "traffic_source": traffic_src,
                    "algorithmic_flops": up_flops, "avg_launch_ms": stages[up_name]}
        if "scattered_gemm" in stages:
            down = 2.0 * L * H * I / (stages["scattered_gemm"] * 1e-3) / 1e12
            roofline["down_gemm_tflops"] = down
            roofline["both_gemms_frac"] = flops / ((stages[up_name] + stages["scattered_gemm"]) * 1e-3) / 1e12 / peak

    out = {
        "metric": metric_name(w) + (f" ({T} tokens)" if args.tokens is not None else ""),
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("bf16 activations, fp8-e4m3 weights" if w.fp8 else {torch.float32: "f32", torch.bfloat16: "bf16",
                  torch.float16: "f16"}[w.dtype]), "data": "synthetic",
        "config": {"workload": w.name, "tokens": T, "hidden": H, "experts": E, "top_k": k, "intermediate": I,
                   "expert_load": "zipf(1.1) first-choice" if w.zipf_s else "near-uniform",
                   "experts_touched": touched, "max_over_min_load": float(counts.max()) / max(1.0, float(counts.min())),
                   **({"fp8_weight_layout": "row-major" if args.fp8_row_major else "streamed tiles"} if w.fp8 else {})},
        "layer_tflops": flops / (elapsed / args.steps) / 1e12,
        "layer_hbm_frac": layer_algorithmic_bytes(w, touched) / (elapsed / args.steps) / 1e9 / PEAK_HBM_GBS,
        "stages_ms": stages,
        "roofline": roofline,
    }
    default_extras = w.name == "granite-3b-a800m" and not args.no_other_workloads and args.tokens is None
    if w.fp8:
        out.update(measure_latency(m, x))
    if default_extras:
        out["ceilings"] = measure_ceilings(w, inputs, device)
        out["block_fusion"] = measure_block_fusion(m, x, w)
    if args.backward or default_extras:
        out["training"] = measure_training(m, x, w, args.steps, full=args.backward)
    if default_extras:
        del m, x
        torch.cuda.empty_cache()
        out["workloads"] = {n: measure_compact(n, device) for n in oracle.WORKLOADS if n != w.name}
        out["routing_stage"] = measure_routing_stage(device)
    if graph_ms is not None:
        out["ms_per_step_graph_replay"] = graph_ms
    if not args.no_cpu_baseline:
        sample = args.cpu_sample_tokens or min(T, 32768 if w.I <= 2048 else 8192)
        out["cpu_baseline"] = cpu_baseline(w, inputs, sample)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
