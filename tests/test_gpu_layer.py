"""End-to-end parity of the MoE module's kernel branch against the CPU oracle.

Routing (expert indices, counts, sort order) must be bit-exact given the same logits; the layer
output must be within rtol = atol = 2e-2 of the fp32 oracle for 16-bit dtypes, and within the
reference's own fp32 tolerance (rtol 1e-3 / atol 2e-4, scattermoe_test.py:38-48) for fp32.
"""

import pytest
import torch

from oracle import moe_oracle as oracle

from _parity import assert_close_scaled, workload_inputs

pytestmark = pytest.mark.gpu


def _build(w, inputs, device, fp8=False):
    from dolomite_engine_amd import MoE

    m = MoE(hidden_size=w.H, intermediate_size=w.I, shared_intermediate_size=None, num_experts=w.E,
            num_experts_per_tok=w.k, activation_function="swiglu", add_bias=False, dropout=0.0,
            init_method="normal", initializer_range=0.02, m_width=None, num_layers=1,
            use_padding_free_transformer=True)
    m = m.to(w.dtype)
    with torch.no_grad():
        m.gate.weight.copy_(inputs["gate_w"])
        if not fp8:
            m.c_fc.weight.copy_(inputs["w_fc"])
            m.c_proj.weight.copy_(inputs["w_proj"])
    m = m.to(device).eval()
    if fp8:  # in the layout the module itself chooses when it quantises (streamed tiles)
        m.c_fc.set_fp8_weight(inputs["w_fc"].to(device), inputs["fc_scale"].to(device), w.dtype, tiled=True, glu=True)
        m.c_proj.set_fp8_weight(inputs["w_proj"].to(device), inputs["proj_scale"].to(device), w.dtype, tiled=True,
                                glu=False)
    if inputs["bias"] is not None:
        m.router_logit_bias = inputs["bias"].to(device)
    return m


def _check_layer(w, T, device, tol):
    from dolomite_engine_amd import Kernel, enable_kernels, ops

    inputs = workload_inputs(w.name, T) if w.name in oracle.WORKLOADS else oracle.make_inputs(w, T=T)
    m = _build(w, inputs, device, fp8=w.fp8)
    x = inputs["x"].to(device)
    print(f"layer {w.name} T={T}", flush=True)
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        y = m(x)
        # routing as the module computed it, with the logits it used
        if ops.router_fused_supported(x, w.E, w.k):
            logits, gates, idx = ops.router_fused(x, m.gate.weight, w.k, bias=m.router_logit_bias, return_logits=True)
        else:
            logits, gates, idx = m._compute_routing_weights(x)
        se, ss, off = ops.sort_bin(idx, w.E)
    assert y.shape == x.shape and y.dtype == x.dtype

    ref = oracle.moe_forward(inputs["x"], inputs["gate_w"], inputs["w_fc"], inputs["w_proj"], w.k,
                             bias=inputs["bias"], logits=logits.cpu(),
                             w_fc_scale=inputs["fc_scale"], w_proj_scale=inputs["proj_scale"])
    # routing: bit-exact on the same logits
    assert torch.equal(idx.cpu().long(), ref.experts)
    assert torch.equal(se.cpu().long(), ref.sorted_expert_idxs)
    assert torch.equal(ss.cpu().long(), ref.sorted_scattered_idxs)
    assert torch.equal(off.cpu().long(), ref.expert_offsets)
    # logits: the device GEMM agrees with the oracle GEMM to one rounding step of the model dtype
    own_logits = oracle.router_logits(inputs["x"], inputs["gate_w"], inputs["bias"])
    step = {torch.float32: 1e-5, torch.bfloat16: 1.6e-2, torch.float16: 2e-3}[w.dtype]
    torch.testing.assert_close(logits.cpu().float(), own_logits.float(), rtol=step, atol=step)
    # Routing on the device's logits against routing on the CPU's logits.  Both GEMMs accumulate in fp32 and round
    # once, so a logit differs only where its exact value sits within the fp32 summation error (about 1e-6
    # relative) of a rounding boundary of the model dtype: a row can be routed differently only if such a logit is
    # one of its k-th / (k+1)-th pair.  On these seeded workloads that happens for no row.
    differs = (oracle.topk_canonical(own_logits, w.k)[1] != ref.experts).any(dim=1)
    print(f"  rows whose routing differs between device logits and CPU logits: {int(differs.sum())} of {differs.numel()}")
    assert int(differs.sum()) == 0
    # output: the stated tolerance and bounds relative to the size of the output
    assert_close_scaled(y, ref.y, w.dtype, what=f"{w.name} T={T}", **tol)
    return y


def test_layer_tiny_fp32(device):
    w = oracle.WORKLOADS["tiny-fp32"]
    _check_layer(w, w.T, device, dict(rtol=1e-3, atol=2e-4))


@pytest.mark.parametrize("name,T", [("granite-1b-a400m", 2048), ("granite-3b-a800m", 2048), ("decode-fp8", 64)])
def test_layer_16bit(device, name, T):
    w = oracle.WORKLOADS[name]
    _check_layer(w, T, device, dict(rtol=2e-2, atol=2e-2))


def test_layer_fp8_many_rows_per_expert(device):
    """fp8 expert weights at a prefill-sized batch (192 rows per expert): the fp8 calls run on the grouped GEMM's tile
    kernels instead of the streaming kernels; same contract against the oracle as the decode batch."""
    import dataclasses

    w = dataclasses.replace(oracle.WORKLOADS["decode-fp8"], E=8, k=2, H=512, I=256, name="fp8-prefill")
    _check_layer(w, 768, device, dict(rtol=2e-2, atol=2e-2))


@pytest.mark.parametrize("H,I", [(264, 256), (256, 152), (72, 40)])
def test_layer_fp8_sizes_not_multiples_of_16(device, H, I):
    """fp8 expert weights with a hidden or intermediate size that the fp8 kernels do not read (they take the
    weights 16 at a time): the module widens the weights for the call and runs the 16-bit kernels; same contract
    against the oracle."""
    import dataclasses

    from dolomite_engine_amd import ops

    w = dataclasses.replace(oracle.WORKLOADS["decode-fp8"], E=8, k=2, H=H, I=I, name="fp8-odd-sizes")
    ops._WARNED.discard(("fp8_widened", H, I))  # (the warning is given once per process and shape)
    with pytest.warns(RuntimeWarning, match="multiples of 16"):
        _check_layer(w, 300, device, dict(rtol=2e-2, atol=2e-2))


def test_layer_mixtral_shape_reduced_experts(device):
    """Mixtral-shape contraction sizes (H=4096, I=14336) with 2 experts so the CPU oracle stays small."""
    import dataclasses

    w = dataclasses.replace(oracle.WORKLOADS["mixtral"], E=2, k=2, name="mixtral-2e")
    _check_layer(w, 256, device, dict(rtol=2e-2, atol=2e-2))


def test_layer_reference_test_shape_generic_activation(device):
    """The reference's own scattermoe test shape (H=32, E=8, k=8, I=128, gelu_pytorch_tanh, T=15):
    the non-GLU kernel path must equal the eager branch of the same module."""
    from dolomite_engine_amd import Kernel, MoE, enable_kernels

    torch.manual_seed(1234)
    # initializer_range 0.15 instead of the reference config's 0.02: the raw layer outputs are then of order 1, like
    # the LM-head logits the reference's test compares, so its absolute tolerances (scattermoe_test.py:38-48: fp32
    # 1e-3 / 2e-4, fp16 atol 2.5e-4, bf16 atol 2e-3 -- the latter two widened to the rounding of an O(1) result of
    # this depth) mean something here
    for dtype, tol in [(torch.float32, dict(rtol=1e-3, atol=2e-4)), (torch.float16, dict(rtol=4e-3, atol=2e-3)),
                       (torch.bfloat16, dict(rtol=2e-2, atol=1e-2))]:
        m = MoE(hidden_size=32, intermediate_size=128, shared_intermediate_size=None, num_experts=8,
                num_experts_per_tok=8, activation_function="gelu_pytorch_tanh", add_bias=False, dropout=0.0,
                init_method="normal", initializer_range=0.15, m_width=None, num_layers=1,
                use_padding_free_transformer=False).to(dtype).to(device).eval()
        x = torch.randn(3, 5, 32, device=device, dtype=dtype)
        with torch.no_grad():
            eager = m(x)
            with enable_kernels([Kernel.scattermoe]):
                fast = m(x)
            # fp32 evaluation of the same module from the same (rounded) parameters: what both branches approximate
            exact = m.float()(x.float())
            m.to(dtype)
        assert exact.abs().max() > 0.3, "outputs must be large compared with the absolute tolerances"
        assert_close_scaled(fast, exact, dtype, what=f"generic activation {dtype}", **tol)
        torch.testing.assert_close(fast.float(), eager.float(), **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_layer_edge_batches(device, dtype):
    """Batches the tile and chunk sizes do not divide: no token at all, one token, the reference test's 15 tokens
    (test_common.py:96-170), 17, a (batch, sequence, hidden) input and a non-contiguous view of a wider tensor; every
    one against the oracle on the same logits, and the empty batch returns an empty tensor of the input's shape."""
    import dataclasses

    from dolomite_engine_amd import Kernel, enable_kernels, ops

    w = dataclasses.replace(oracle.WORKLOADS["tiny-fp32"], dtype=dtype, H=64, I=96, E=8, k=2, name="edge")
    inputs = oracle.make_inputs(w, T=40)
    m = _build(w, inputs, device)
    tol = dict(rtol=1e-3, atol=2e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)

    def run(x_dev):
        with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
            y = m(x_dev)
            # the logits of the call the forward itself makes for this batch
            flat = x_dev.reshape(-1, w.H)
            if flat.shape[0] and m._use_fused_router(flat) and ops.router_fused_sort_supported(flat, w.E, w.k):
                logits = ops.router_fused_sort(flat, m.gate.weight, w.k, bias=m.router_logit_bias, return_logits=True)[0]
            elif flat.shape[0] and ops.router_fused_supported(flat, w.E, w.k):
                logits = ops.router_fused(flat, m.gate.weight, w.k, bias=m.router_logit_bias, return_logits=True)[0]
            else:
                logits = m._compute_routing_weights(flat)[0]
        return y, logits

    for T in (0, 1, 15, 17):
        print(f"edge batch T={T} {dtype}", flush=True)
        x = inputs["x"][:T].contiguous()
        y, logits = run(x.to(device))
        assert y.shape == x.shape and y.dtype == dtype
        if T == 0:
            continue
        ref = oracle.moe_forward(x, inputs["gate_w"], inputs["w_fc"], inputs["w_proj"], w.k, logits=logits.cpu())
        assert_close_scaled(y, ref.y, dtype, what=f"edge T={T}", **tol)

    print(f"edge batch 3-D {dtype}", flush=True)
    x3 = inputs["x"][:21].reshape(3, 7, w.H).contiguous()
    m.use_padding_free_transformer = False  # (batch, sequence, hidden) in and out, moe.py:213-216, 228-229
    y3, logits = run(x3.to(device))
    m.use_padding_free_transformer = True
    assert y3.shape == x3.shape
    ref = oracle.moe_forward(x3.reshape(21, w.H), inputs["gate_w"], inputs["w_fc"], inputs["w_proj"], w.k, logits=logits.cpu())
    assert_close_scaled(y3.reshape(21, w.H), ref.y, dtype, what="edge 3-D", **tol)

    print(f"edge batch non-contiguous {dtype}", flush=True)
    wide = torch.zeros(40, 2 * w.H, dtype=dtype)
    wide[:, : w.H] = inputs["x"]
    view = wide.to(device)[:, : w.H]
    assert not view.is_contiguous()
    yv, logits = run(view)
    ref = oracle.moe_forward(inputs["x"], inputs["gate_w"], inputs["w_fc"], inputs["w_proj"], w.k, logits=logits.cpu())
    assert_close_scaled(yv, ref.y, dtype, what="edge non-contiguous", **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_layer_shared_experts(device, dtype, monkeypatch):
    """Shared experts (moe.py:311-315) on the kernel branch run on the grouped-GEMM kernels in every dtype: the
    module's two shared linear layers must not be called at all."""
    from dolomite_engine_amd import Kernel, MoE, enable_kernels

    torch.manual_seed(7)
    m = MoE(hidden_size=128, intermediate_size=64, shared_intermediate_size=96, num_experts=8,
            num_experts_per_tok=2, activation_function="swiglu", add_bias=False, dropout=0.0, init_method="normal",
            initializer_range=0.05, m_width=None, num_layers=1, use_padding_free_transformer=True)
    m = m.to(dtype).to(device).eval()
    x = torch.randn(300, 128, device=device, dtype=dtype)

    def refuse(*a, **k):
        raise AssertionError("the shared experts went through torch's linear layer on the kernel branch")

    monkeypatch.setattr(m.c_fc_shared, "forward", refuse)
    monkeypatch.setattr(m.c_proj_shared, "forward", refuse)
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        y = m(x)
        # the logits as the module's router kernel produced them (fp32 sums differ by order: route on these)
        from dolomite_engine_amd import ops
        logits = ops.router_fused(x, m.gate.weight, 2, return_logits=True)[0]
    ref = oracle.moe_forward(x.cpu(), m.gate.weight.cpu(), m.c_fc.weight.cpu(), m.c_proj.weight.cpu(), 2,
                             logits=None if logits is None else logits.cpu(),
                             shared_fc=m.c_fc_shared.weight.cpu(), shared_proj=m.c_proj_shared.weight.cpu())
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-3, atol=2e-4)
    assert_close_scaled(y, ref.y, dtype, what="shared experts", **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shared_size", [None, 96])
def test_layer_block_tail(device, dtype, shared_size):
    """Shared experts, m_residual and the residual folded into the combine pass: bit-identical to the same
    module followed by the separate torch operations, and within tolerance of the fp32 oracle."""
    from dolomite_engine_amd import Kernel, MoE, enable_kernels

    torch.manual_seed(11)
    m = MoE(hidden_size=128, intermediate_size=64, shared_intermediate_size=shared_size, num_experts=8,
            num_experts_per_tok=2, activation_function="swiglu", add_bias=False, dropout=0.0, init_method="normal",
            initializer_range=0.05, m_width=None, num_layers=1, use_padding_free_transformer=True)
    m = m.to(dtype).to(device).eval()
    x = torch.randn(333, 128, device=device, dtype=dtype)
    res = torch.randn(333, 128, device=device, dtype=dtype)
    scale = 0.22
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        fused = m(x, residual=res, residual_scale=scale)
        plain = m(x)                      # shared experts (if any) are folded in here too
        unfused = plain * scale + res     # the block's own two operations
        only_scale = m(x, residual_scale=scale)
        only_res = m(x, residual=res)
    assert torch.equal(fused, unfused)
    assert torch.equal(only_scale, plain * scale)
    assert torch.equal(only_res, plain + res)
    kw = {} if shared_size is None else dict(shared_fc=m.c_fc_shared.weight.cpu(), shared_proj=m.c_proj_shared.weight.cpu())
    ref = oracle.moe_forward(x.cpu(), m.gate.weight.cpu(), m.c_fc.weight.cpu(), m.c_proj.weight.cpu(), 2,
                             residual=res.cpu(), residual_scale=scale, **kw)
    torch.testing.assert_close(fused.cpu().float(), ref.y, rtol=2e-2, atol=2e-2)
    # the eager branch takes the same arguments
    with torch.no_grad():
        eager = m(x, residual=res, residual_scale=scale)
    torch.testing.assert_close(eager.float(), fused.float(), rtol=2e-2, atol=2e-2)


def test_layer_with_pre_norm(device):
    """ln_2 folded into the layer: same routing and (to rounding of x_norm) same output as RMSNorm followed by the
    layer, on the kernel branch and on the eager branch; and close to the fp32 oracle of norm + layer."""
    from dolomite_engine_amd import Kernel, MoE, enable_kernels

    torch.manual_seed(3)
    m = MoE(hidden_size=256, intermediate_size=128, shared_intermediate_size=None, num_experts=8,
            num_experts_per_tok=2, activation_function="swiglu", add_bias=False, dropout=0.0, init_method="normal",
            initializer_range=0.05, m_width=None, num_layers=1, use_padding_free_transformer=True)
    m = m.to(torch.bfloat16).to(device).eval()
    h = (torch.randn(777, 256, device=device) * 3).bfloat16()
    lnw = (1 + 0.2 * torch.randn(256, device=device)).bfloat16()
    res = torch.randn(777, 256, device=device).bfloat16()
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        fused = m(h, residual=res, residual_scale=0.5, pre_norm=(lnw, 1e-5))
        unfused = m(torch.nn.functional.rms_norm(h, (256,), lnw, 1e-5), residual=res, residual_scale=0.5)
    with torch.no_grad():
        eager = m(h, residual=res, residual_scale=0.5, pre_norm=(lnw, 1e-5))
    torch.testing.assert_close(fused.float(), unfused.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(fused.float(), eager.float(), rtol=2e-2, atol=2e-2)
    xn = oracle.rmsnorm(h.cpu(), lnw.cpu(), 1e-5)
    ref = oracle.moe_forward(xn, m.gate.weight.cpu(), m.c_fc.weight.cpu(), m.c_proj.weight.cpu(), 2,
                             residual=res.cpu(), residual_scale=0.5)
    torch.testing.assert_close(fused.cpu().float(), ref.y, rtol=2e-2, atol=2e-2)


def test_combine_block_tail_matches_separate_ops(device):
    """mi_moe_combine_block_tail == mi_moe_combine followed by torch's add / mul / add, bit for bit, for
    every subset of the three optional steps (vector and scalar kernels)."""
    from dolomite_engine_amd import ops

    g = torch.Generator().manual_seed(5)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        for T, k, H in ((70, 8, 1536), (33, 3, 100)):
            o = torch.randn(T * k, H, generator=g).to(dtype).to(device)
            gates = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype).to(device)
            shared = torch.randn(T, H, generator=g).to(dtype).to(device)
            res = torch.randn(T, H, generator=g).to(dtype).to(device)
            base = ops.combine(o, gates)
            for use_sh in (False, True):
                for scale in (None, 0.3):
                    for use_res in (False, True):
                        got = ops.combine(o, gates, shared if use_sh else None, res if use_res else None, scale)
                        want = base
                        if use_sh:
                            want = want + shared
                        if scale is not None:
                            want = want * scale
                        if use_res:
                            want = want + res
                        assert torch.equal(got, want), (dtype, T, k, H, use_sh, scale, use_res)


@pytest.mark.parametrize("name,T", [("decode-fp8", 64), ("granite-1b-a400m", 512)])
def test_layer_under_hip_graph_capture(device, name, T):
    """The kernel branch is capture-safe: no host synchronisation, no memset nodes, outputs from the caching
    allocator.  A captured forward is replayed several times with new inputs, with eager work and
    synchronisations in between, and every replay must equal the eager result bit for bit."""
    from dolomite_engine_amd import Kernel, enable_kernels

    w = oracle.WORKLOADS[name]
    inputs = oracle.make_inputs(w, T=T)
    m = _build(w, inputs, device, fp8=w.fp8)
    g = torch.Generator().manual_seed(5)
    xs = [torch.randn(T, w.H, generator=g).to(w.dtype).to(device) for _ in range(4)]
    static_x = xs[0].clone()
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                m(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = m(static_x)
        for i, x in enumerate(xs * 2):
            eager = m(x)
            torch.cuda.synchronize()
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, eager), f"replay {i}"


def test_low_level_ops_record_no_gradient(device):
    """The tensor-level kernel wrappers are not differentiable and say so (the differentiable compositions are
    the module and autograd.py)."""
    from dolomite_engine_amd import ops

    x = torch.randn(8, 64, device=device, dtype=torch.bfloat16, requires_grad=True)
    w = torch.randn(4, 32, 64, device=device, dtype=torch.bfloat16)
    ss = torch.arange(8, device=device, dtype=torch.int32)
    off = torch.tensor([2, 4, 6, 8], device=device, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="forward-only"):
        ops.scattered_gemm(x, w, 1, ss, off, False, True)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, dict(rtol=2e-3, atol=2e-5)), (torch.bfloat16, dict(rtol=5e-2, atol=2e-2))])
@pytest.mark.parametrize("shared", [None, 64])
@pytest.mark.parametrize("activation", ["swiglu", "swiglu-recompute", "gelu_pytorch_tanh", "geglu"])
def test_training_gradients_match_eager_branch(device, dtype, tol, shared, activation):
    """Training through the kernel branch: output, aux loss and every gradient (input, router, both expert
    weight tensors, shared experts) against torch autograd through the eager branch of the same module.
    swiglu takes the fused expert function, the other activations the differentiable scattered_experts with the
    activation in torch between the two grouped GEMMs."""
    from dolomite_engine_amd import Kernel, MoE, enable_kernels
    from dolomite_engine_amd.loss import clear_aux_loss, get_aux_loss

    # "swiglu": the pre-activation of the up-projection is kept for the backward; "swiglu-recompute": recomputed there
    keep = activation != "swiglu-recompute"
    activation = activation.split("-")[0]
    torch.manual_seed(21)
    m = MoE(hidden_size=128, intermediate_size=64, shared_intermediate_size=shared, num_experts=8,
            num_experts_per_tok=2, activation_function=activation, add_bias=False, dropout=0.0, init_method="normal",
            initializer_range=0.1, m_width=None, num_layers=1, use_padding_free_transformer=True)
    m = m.to(dtype).to(device).train()
    m.keep_preactivation = keep
    x0 = torch.randn(300, 128, device=device, dtype=dtype)
    dy = torch.randn(300, 128, device=device, dtype=dtype)

    def run(kernels):
        m.zero_grad(set_to_none=True)
        clear_aux_loss()
        x = x0.clone().requires_grad_(True)
        if kernels:
            with enable_kernels([Kernel.scattermoe]):
                y = m(x)
        else:
            y = m(x)
        aux = get_aux_loss()
        ((y * dy).sum() + 0.01 * aux).backward()
        grads = {n: p.grad.detach().clone() for n, p in m.named_parameters()}
        return y.detach(), aux.detach(), x.grad.detach(), grads

    y_e, aux_e, dx_e, g_e = run(False)
    y_k, aux_k, dx_k, g_k = run(True)
    torch.testing.assert_close(y_k.float(), y_e.float(), **tol)
    # the kernel branch computes the aux loss in fp32, the eager branch in the model dtype
    torch.testing.assert_close(aux_k.float(), aux_e.float(), rtol=1e-4 if dtype == torch.float32 else 2e-2, atol=1e-5)
    # relative to the largest entry, like the parameter gradients below
    dx_scale = dx_e.float().abs().max().clamp_min(1e-6)
    torch.testing.assert_close(dx_k.float() / dx_scale, dx_e.float() / dx_scale, rtol=tol["rtol"], atol=tol["rtol"] / 4)
    assert set(g_k) == set(g_e)
    for n in g_e:
        scale = g_e[n].float().abs().max().clamp_min(1e-6)
        # relative to the largest entry of the gradient: both branches round bf16 intermediates differently
        torch.testing.assert_close(g_k[n].float() / scale, g_e[n].float() / scale, rtol=tol["rtol"], atol=tol["rtol"]), n


@pytest.mark.parametrize("name", ["granite-1b-a400m", "granite-3b-a800m", "mixtral"])
def test_full_size_properties(device, name):
    """Full benchmark sizes: size-independent properties instead of a CPU recomputation.

    * routing invariants: every token has k distinct experts, sorted ids non-decreasing, the scatter
      index is a permutation, offsets == cumsum(bincount);
    * the layer is linear in the down-projection weights and in the gates: scaling c_proj by 2
      doubles the output (exactly, powers of two);
    * a random sample of tokens is recomputed by the oracle."""
    from dolomite_engine_amd import Kernel, enable_kernels, ops

    w = oracle.WORKLOADS[name]
    inputs = workload_inputs(name)
    m = _build(w, inputs, device)
    x = inputs["x"].to(device)
    print(f"full size {name}", flush=True)
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        y = m(x)
        logits, gates, idx = ops.router_fused(x, m.gate.weight, w.k, bias=m.router_logit_bias, return_logits=True)
        se, ss, off = ops.sort_bin(idx, w.E)
        m.c_proj.weight.mul_(2.0)
        y2 = m(x)
        m.c_proj.weight.mul_(0.5)
    L = w.T * w.k
    idx_c = idx.cpu().long()
    assert (idx_c.sort(dim=1).values.diff(dim=1) > 0).all(), "experts of a token must be distinct"
    assert (se.diff() >= 0).all()
    assert torch.equal(ss.sort().values.cpu().long(), torch.arange(L))
    assert torch.equal(off.cpu().long(), torch.bincount(idx_c.flatten(), minlength=w.E).cumsum(0))
    assert torch.equal(se.cpu().long(), idx_c.flatten()[ss.cpu().long()])
    assert torch.equal(y2.float(), 2 * y.float())
    # sampled tokens against the oracle (same logits -> same routing)
    g = torch.Generator().manual_seed(0)
    sample = torch.randperm(w.T, generator=g)[:256 if w.I <= 4096 else 48]  # the oracle runs on the host
    ref = oracle.moe_forward(inputs["x"][sample], inputs["gate_w"], inputs["w_fc"], inputs["w_proj"], w.k,
                             bias=inputs["bias"], logits=logits.cpu()[sample])
    assert torch.equal(idx_c[sample], ref.experts)
    assert_close_scaled(y.cpu()[sample], ref.y, w.dtype, rtol=2e-2, atol=2e-2, what=f"{name} sampled tokens")
    if w.zipf_s is not None:
        counts = torch.bincount(idx_c.flatten(), minlength=w.E).double()
        print("  per-expert load (sorted):", (counts.sort(descending=True).values / L).numpy().round(4)[:8])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_training_and_inference_route_tied_rows_alike(device, dtype):
    """Logits on a coarse grid (many exact ties, also between the k-th and the (k+1)-th): the kernel branch must
    pick the canonical experts (value descending, expert index ascending; moe.py:338-344 leaves the order to
    torch.topk) in train() mode with gradients as it does in eval() mode, and the router's gradient must reach
    the gate weights."""
    from dolomite_engine_amd import Kernel, MoE, enable_kernels

    T, H, E, k = 257, 64, 40, 8
    m = MoE(hidden_size=H, intermediate_size=64, shared_intermediate_size=None, num_experts=E,
            num_experts_per_tok=k, activation_function="swiglu", add_bias=False, dropout=0.0, init_method="normal",
            initializer_range=0.02, m_width=None, num_layers=1, use_padding_free_transformer=True).to(dtype).to(device)
    g = torch.Generator().manual_seed(9)
    with torch.no_grad():  # entries in {-1, 0, 1} x {-0.5, 0, 0.5}: every logit is a multiple of 0.5, exactly
        m.gate.weight.copy_((torch.randint(-1, 2, (E, H), generator=g) * 0.5).to(dtype))
    x = torch.randint(-1, 2, (T, H), generator=g).to(dtype).to(device)
    logits_ref = (x.cpu().float() @ m.gate.weight.detach().cpu().float().t()).to(dtype)
    srt = logits_ref.float().sort(dim=-1, descending=True).values
    assert (srt[:, k - 1] == srt[:, k]).float().mean() > 0.2, "the test needs ties at the selection boundary"
    _, want = oracle.topk_canonical(logits_ref, k)

    with enable_kernels([Kernel.scattermoe]):
        m.train()
        xg = x.clone().requires_grad_(True)
        logits, gates, idx = m._compute_routing_weights(xg)
        assert torch.equal(logits.detach().cpu(), logits_ref)
        assert torch.equal(idx.cpu().long(), want), "training-mode routing is not the canonical one"
        weight = torch.arange(k, device=device, dtype=torch.float32)
        (gates.float() * weight).sum().backward()
        assert m.gate.weight.grad is not None and m.gate.weight.grad.abs().sum() > 0
        assert xg.grad is not None and xg.grad.abs().sum() > 0
        m.eval()
        with torch.no_grad():
            _, gates_eval, idx_eval = m._compute_routing_weights(x)
    assert torch.equal(idx_eval.cpu().long(), want), "inference-mode routing is not the canonical one"
    ulp = {torch.bfloat16: 8e-3, torch.float32: 2e-6}[dtype]  # torch's softmax and the kernel's differ by a rounding
    torch.testing.assert_close(gates.detach().float(), gates_eval.float(), rtol=ulp, atol=ulp * 0.1)


@pytest.mark.parametrize("seed", list(range(16)))
def test_training_random_shapes(device, seed):
    """Training through the kernel branch at random shapes (token counts around the kernels' tile and dispatch
    boundaries, hidden and intermediate sizes that are multiples of 8 only, 2 to 72 experts, with and without
    shared experts, the pre-activation kept or recomputed): output, aux loss and every gradient against torch
    autograd through the eager branch of the same module, each relative to its largest entry.  k >= 2 and no fp16:
    with one expert per token only the aux loss reaches the gate weights, and the eager branch's 16-bit aux loss
    is the less exact side of that comparison."""
    import random

    from dolomite_engine_amd import Kernel, MoE, enable_kernels
    from dolomite_engine_amd.loss import clear_aux_loss, get_aux_loss

    rng = random.Random(1000 + seed)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float32])
    T = rng.choice([2, 15, 17, 63, 65, 300, 321, 1000, 1025, 2500, 4100]) if rng.random() < 0.5 else rng.randint(2, 3000)
    H = 8 * rng.randint(2, 160) if rng.random() < 0.7 else 32 * rng.randint(1, 48)
    E = rng.choice([2, 3, 7, 8, 16, 17, 32, 40, 64, 65, 72])
    k = rng.randint(2, min(E, 8))
    I = 8 * rng.randint(1, 96) if rng.random() < 0.7 else 64 * rng.randint(1, 12)
    shared = rng.choice([None, None, 8 * rng.randint(1, 40)])
    activation = rng.choice(["swiglu", "swiglu", "swiglu", "gelu_pytorch_tanh", "geglu"])
    keep = rng.random() < 0.6
    print(f"training {dtype} T={T} H={H} E={E} k={k} I={I} shared={shared} {activation} keep={keep}", flush=True)
    torch.manual_seed(seed)
    m = MoE(hidden_size=H, intermediate_size=I, shared_intermediate_size=shared, num_experts=E,
            num_experts_per_tok=k, activation_function=activation, add_bias=False, dropout=0.0, init_method="normal",
            initializer_range=0.1, m_width=None, num_layers=1, use_padding_free_transformer=True)
    m = m.to(dtype).to(device).train()
    m.keep_preactivation = keep
    x0 = torch.randn(T, H, device=device, dtype=dtype)
    dy = torch.randn(T, H, device=device, dtype=dtype)
    with torch.no_grad():
        idx_e = m._compute_routing_weights(x0)[2].long().sort(dim=1).values
        with enable_kernels([Kernel.scattermoe]):
            idx_k = m._compute_routing_weights(x0)[2].long().sort(dim=1).values
    if not torch.equal(idx_e, idx_k):  # a logit on a rounding boundary of the model dtype: the branches route apart
        pytest.skip("the two branches' logits round a selection boundary differently on this seed")

    def run(kernels):
        m.zero_grad(set_to_none=True)
        clear_aux_loss()
        x = x0.clone().requires_grad_(True)
        if kernels:
            with enable_kernels([Kernel.scattermoe]):
                y = m(x)
        else:
            y = m(x)
        aux = get_aux_loss()
        ((y * dy).sum() + 0.01 * aux).backward()
        return y.detach(), aux.detach(), x.grad.detach(), {n: p.grad.detach().clone() for n, p in m.named_parameters()}

    y_e, aux_e, dx_e, g_e = run(False)
    y_k, aux_k, dx_k, g_k = run(True)
    tol = {torch.float32: 2e-3, torch.bfloat16: 5e-2}[dtype]
    torch.testing.assert_close(aux_k.float(), aux_e.float(), rtol=1e-4 if dtype == torch.float32 else 2e-2, atol=1e-5)
    assert set(g_k) == set(g_e)
    for name, got, want in [("y", y_k, y_e), ("dx", dx_k, dx_e)] + [(n, g_k[n], g_e[n]) for n in g_e]:
        scale = want.float().abs().max().clamp_min(1e-6)
        err = ((got.float() - want.float()).abs().max() / scale).item()
        assert err <= tol, f"{name}: {err:.3e} of the largest entry"
