"""GPU parity of the element-wise backward kernels against fp32 formulas evaluated with torch autograd on the CPU.

The expected values come from differentiating the forward definitions (``up * silu(gate)``,
activations/glu.py:42-43, and the gate-weighted sum of moe.py:282-290) with autograd in fp32, not from a
retyped derivative; results are 16-bit so the comparison is at the rounding of the output dtype.
"""

import pytest
import torch
import torch.nn.functional as F

from _parity import assert_close_scaled

pytestmark = pytest.mark.gpu


def _ops():
    from dolomite_engine_amd import ops

    return ops


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("L,I,k", [(1, 8, 1), (36, 64, 2), (512, 512, 8), (4098, 1408, 6), (30, 12, 3)])
@pytest.mark.parametrize("routed", [False, True])
def test_swiglu_backward(device, dtype, L, I, k, routed):
    """d_h, g * a and the router-weight gradient against autograd through z = sum_i g_i <c_i, up_i * silu(gate_i)>
    (c = d_act plays the role of the upstream gradient w_proj^T dy)."""
    if I % 8 and dtype != torch.float32:
        pytest.skip("a row of 16-bit values must be whole 16-byte chunks")
    g = torch.Generator().manual_seed(L * 31 + I)
    h = (torch.randn(L, 2 * I, generator=g) * 2).to(dtype)
    d_act = torch.randn(L, I, generator=g).to(dtype)
    gates = torch.rand(L // k, k, generator=g).to(dtype) if routed else None
    ss = torch.randperm(L, generator=g).to(torch.int32) if routed else None

    hf = h.float().clone().requires_grad_(True)
    a = hf[:, :I] * F.silu(hf[:, I:])
    if routed:
        gf = gates.float().clone().requires_grad_(True)
        g_rows = gf.reshape(-1)[ss.long()].unsqueeze(-1)
    else:
        g_rows = 1.0
    (g_rows * d_act.float() * a).sum().backward()

    d_h, act_g, d_gates = _ops().swiglu_backward(
        h.to(device), d_act.to(device), None if gates is None else gates.to(device),
        None if ss is None else ss.to(device), want_act=True, want_gate_grad=routed)
    assert d_h.dtype == dtype and tuple(d_h.shape) == (L, 2 * I)
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2e-6}[dtype]
    torch.testing.assert_close(d_h.cpu().float(), hf.grad, rtol=2 * eps, atol=1e-6)
    torch.testing.assert_close(act_g.cpu().float(), (g_rows * a).detach(), rtol=2 * eps, atol=1e-6)
    if routed:
        assert tuple(d_gates.shape) == tuple(gates.shape)
        torch.testing.assert_close(d_gates.cpu().float(), gf.grad, rtol=2 * eps, atol=2e-4 * I ** 0.5)
    else:
        assert d_gates is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("L,I", [(1, 8), (77, 136), (1000, 512), (5, 100)])
def test_swiglu_forward(device, dtype, L, I):
    """a = up * silu(gate) of a stored pre-activation against the closed form in fp64 on the same rounded h
    (activations/glu.py:42-43); (5, 100) in a 16-bit dtype takes the torch form inside the wrapper."""
    g = torch.Generator().manual_seed(L + I)
    h = (torch.randn(L, 2 * I, generator=g) * 2).to(dtype)
    got = _ops().swiglu_forward(h.to(device))
    hd = h.double()
    ref = hd[:, :I] * hd[:, I:] * torch.sigmoid(hd[:, I:])
    assert got.shape == (L, I) and got.dtype == dtype
    tol = {torch.float32: 1e-6, torch.float16: 1e-3, torch.bfloat16: 8e-3}[dtype]
    torch.testing.assert_close(got.cpu().double(), ref, rtol=tol, atol=tol)
    assert got.abs().max() > 0.5


def test_swiglu_backward_empty_and_errors(device):
    ops = _ops()
    out, act_g, d_gates = ops.swiglu_backward(torch.empty(0, 32, device=device, dtype=torch.bfloat16),
                                              torch.empty(0, 16, device=device, dtype=torch.bfloat16))
    assert tuple(out.shape) == (0, 32) and act_g is None and d_gates is None
    with pytest.raises(ValueError):
        ops.swiglu_backward(torch.zeros(4, 30, device=device, dtype=torch.bfloat16),
                            torch.zeros(4, 16, device=device, dtype=torch.bfloat16))
    with pytest.raises(ValueError):  # the router-weight gradient needs the router weights
        ops.swiglu_backward(torch.zeros(4, 32, device=device, dtype=torch.bfloat16),
                            torch.zeros(4, 16, device=device, dtype=torch.bfloat16), want_gate_grad=True)
    from dolomite_engine_amd._lib import MiMoeError

    with pytest.raises(MiMoeError):  # fp32: I % 4 != 0
        ops.swiglu_backward(torch.zeros(4, 12, device=device), torch.zeros(4, 6, device=device))
    with pytest.raises(MiMoeError):  # I % 8 != 0
        ops.swiglu_backward(torch.zeros(4, 24, device=device, dtype=torch.bfloat16),
                            torch.zeros(4, 12, device=device, dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,k,H", [(1, 1, 8), (5, 2, 64), (300, 8, 1536), (64, 6, 4096), (1027, 2, 520), (9, 3, 12)])
def test_combine_grad_gates(device, dtype, T, k, H):
    if H % 8 and dtype != torch.float32:
        pytest.skip("a row of 16-bit values must be whole 16-byte chunks")
    g = torch.Generator().manual_seed(T + k + H)
    o = torch.randn(T * k, H, generator=g).to(dtype)
    dy = torch.randn(T, H, generator=g).to(dtype)
    gates = torch.rand(T, k, generator=g).requires_grad_(True)
    y = (gates.unsqueeze(-1) * o.float().view(T, k, H)).sum(dim=1)
    y.backward(dy.float())

    got = _ops().combine_grad_gates(o.to(device), dy.to(device), k)
    assert got.dtype == dtype and tuple(got.shape) == (T, k)
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2e-6}[dtype]
    # an fp32 dot product of H terms rounded once; the absolute term covers cancellation
    torch.testing.assert_close(got.cpu().float(), gates.grad, rtol=2 * eps, atol=1e-4 * H ** 0.5)


def _wgrad_reference(a, b, offsets, a_idx, b_idx):
    """fp64 loop over experts: the definition, with plain matrix products."""
    E = offsets.shape[0]
    out = torch.zeros(E, a.shape[1], b.shape[1], dtype=torch.float64)
    start = 0
    for e, end in enumerate(offsets.tolist()):
        if end > start:
            rows = torch.arange(start, end)
            ar = a[a_idx[rows].long()] if a_idx is not None else a[rows]
            br = b[b_idx[rows].long()] if b_idx is not None else b[rows]
            out[e] = ar.double().t() @ br.double()
        start = end
    return out


WGRAD_CASES = [
    # L, E, M, N, rows_other (rows of the gathered operand)
    (1, 1, 8, 8, 1),
    (33, 3, 16, 24, 9),
    (700, 8, 256, 256, 350),
    (1500, 5, 264, 520, 200),      # ragged column tiles on both operands
    (5000, 40, 512, 128, 625),     # many experts, several row groups per expert
    (2100, 130, 64, 72, 300),      # more experts than one ballot covers
]


def _seeded_counts(L, weights, g):
    """Sizes of E groups that add up to L: L draws from the given weights, from the seeded generator only."""
    draws = torch.multinomial(weights.double(), L, replacement=True, generator=g)
    return torch.bincount(draws, minlength=weights.numel())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("L,E,M,N,rows_other", WGRAD_CASES + [(900, 6, 132, 260, 100)])  # (fp32: multiples of 4)
@pytest.mark.parametrize("gather", ["a", "b", "none", "both"])
def test_grouped_wgrad(device, dtype, L, E, M, N, rows_other, gather):
    g = torch.Generator().manual_seed(L * 7 + E)
    # skewed expert sizes with empty experts in between
    w = torch.rand(E, generator=g).pow(3)
    w[torch.rand(E, generator=g) < 0.25] = 0
    if w.sum() == 0:
        w[0] = 1
    counts = _seeded_counts(L, w, g)
    offsets = counts.cumsum(0).to(torch.int32)
    assert int(offsets[-1]) == L
    ga, gb = gather in ("a", "both"), gather in ("b", "both")
    a = torch.randn(rows_other if ga else L, M, generator=g).to(dtype)
    b = torch.randn(rows_other if gb else L, N, generator=g).to(dtype)
    a_idx = torch.randint(0, rows_other, (L,), generator=g, dtype=torch.int32) if ga else None
    b_idx = torch.randint(0, rows_other, (L,), generator=g, dtype=torch.int32) if gb else None

    got = _ops().grouped_wgrad(a.to(device), b.to(device), offsets.to(device),
                               None if a_idx is None else a_idx.to(device), None if b_idx is None else b_idx.to(device))
    assert got.dtype == dtype and tuple(got.shape) == (E, M, N)
    ref = _wgrad_reference(a, b, offsets, a_idx, b_idx)
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -20}[dtype]
    # fp32 accumulation of up to L products of unit-variance terms, one rounding to the dtype
    torch.testing.assert_close(got.cpu().double(), ref, rtol=2 * eps, atol=2e-5 * max(1.0, counts.max().item()) ** 0.5 + 1e-6)
    # experts without rows get exact zeros
    for e in (counts == 0).nonzero().flatten().tolist():
        assert not got[e].any()


KEEP_CASES = [
    # counts per expert, H, I
    ([5000, 5000, 5000, 5000], 1536, 512),          # interior tiles, a partly filled last round
    ([1, 9000, 0, 300, 12000, 257], 1024, 520),     # ragged experts (row tails), ragged last column tile
    ([700, 0, 650, 900], 256, 128),                 # few tiles, short contraction
    ([40, 30, 20, 10], 256, 64),                    # too few rows per expert for the tile kernel: the two-call path
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("counts,H,I", KEEP_CASES)
def test_up_swiglu_keep(device, dtype, counts, H, I):
    """The training up-projection (activation and pre-activation from one launch) against the two calls it stands
    for: the pre-activation bit for bit (same accumulators, same rounding), the activation formed from the rounded
    pre-activation, equal up to the last place (a reciprocal where the element-wise kernel divides)."""
    ops = _ops()
    g = torch.Generator().manual_seed(sum(counts) + H)
    E, L, k = len(counts), sum(counts), 2
    T = L // k
    assert T * k == L
    off = torch.tensor(counts).cumsum(0).to(torch.int32).to(device)
    ss = torch.randperm(L, generator=g).to(torch.int32).to(device)
    x = torch.randn(T, H, generator=g).to(dtype).to(device)
    w = (torch.randn(E, 2 * I, H, generator=g) * 0.05).to(dtype).to(device)
    print(f"up_swiglu_keep {dtype} counts={counts} H={H} I={I}", flush=True)
    act, h = ops.up_swiglu_keep(x, w, k, ss, off)
    h_ref = ops.scattered_gemm(x, w, k, ss, off, False, True)
    act_ref = ops.swiglu_forward(h_ref)
    assert h.shape == (L, 2 * I) and act.shape == (L, I)
    assert torch.equal(h, h_ref)
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    diff = (act.float() - act_ref.float()).abs()
    assert bool((diff <= act_ref.float().abs() * 2 * eps + 1e-6).all())
    assert (act != act_ref).float().mean().item() < 0.02
    # and against fp32 arithmetic on the same rounded h
    hf = h_ref.float()
    ref = hf[:, :I] * torch.nn.functional.silu(hf[:, I:])
    assert_close_scaled(act, ref, dtype, rtol=2e-2, atol=2e-2, what="up_swiglu_keep")


def test_grouped_wgrad_is_deterministic(device):
    g = torch.Generator().manual_seed(5)
    L, E, M, N = 9000, 6, 256, 512
    a = torch.randn(L, M, generator=g).to(torch.bfloat16).to(device)
    b = torch.randn(L, N, generator=g).to(torch.bfloat16).to(device)
    offsets = torch.tensor([4000, 4000, 4100, 8000, 8990, 9000], dtype=torch.int32, device=device)
    first = _ops().grouped_wgrad(a, b, offsets)
    for _ in range(3):
        assert torch.equal(_ops().grouped_wgrad(a, b, offsets), first)


def test_grouped_wgrad_no_rows(device):
    ops = _ops()
    a = torch.empty(0, 16, dtype=torch.bfloat16, device=device)
    b = torch.empty(0, 8, dtype=torch.bfloat16, device=device)
    out = ops.grouped_wgrad(a, b, torch.zeros(4, dtype=torch.int32, device=device))
    assert tuple(out.shape) == (4, 16, 8) and not out.any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k", [(1, 4, 1), (15, 8, 8), (300, 40, 8), (1000, 64, 6), (129, 130, 2), (4100, 256, 3)])
def test_aux_loss_and_gradient(device, dtype, T, E, k):
    """Value against the oracle's restatement of moe.py:346-369 on the same (rounded) logits, gradient against
    autograd through that restatement; both in fp32, so only the summation order differs."""
    from oracle import moe_oracle as oracle

    g = torch.Generator().manual_seed(T + E * 7 + k)
    logits = (torch.randn(T, E, generator=g) * 1.5).to(dtype)
    idx = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k].contiguous()
    ops = _ops()

    lf = logits.float().clone().requires_grad_(True)
    ref = oracle.switch_aux_loss(lf, idx)
    upstream = 0.37
    (ref * upstream).backward()

    loss_w = ops.aux_loss(logits.to(device), idx.to(device))
    assert loss_w.dtype == torch.float32 and tuple(loss_w.shape) == (1 + E,)
    torch.testing.assert_close(loss_w[0].cpu(), ref.detach(), rtol=2e-5, atol=1e-6)
    d = ops.aux_loss_backward(logits.to(device), loss_w, torch.tensor(upstream, device=device))
    assert d.dtype == dtype and tuple(d.shape) == (T, E)
    eps = {torch.float32: 2e-5, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    # entries are O(1 / T); compare relative to the largest one
    scale = lf.grad.abs().max()
    torch.testing.assert_close(d.cpu().float() / scale, lf.grad / scale, rtol=2 * eps, atol=2 * eps)
    # deterministic
    assert torch.equal(ops.aux_loss(logits.to(device), idx.to(device)), loss_w)


def test_aux_loss_autograd_function(device):
    from dolomite_engine_amd.autograd import SwitchAuxLoss
    from oracle import moe_oracle as oracle

    g = torch.Generator().manual_seed(3)
    logits = torch.randn(200, 16, generator=g)
    idx = torch.rand(200, 16, generator=g).argsort(dim=1)[:, :4].contiguous()
    a = logits.clone().to(device).requires_grad_(True)
    loss = SwitchAuxLoss.apply(a, idx.to(device))
    assert loss.dim() == 0 and loss.dtype == torch.float32
    (loss * 2.0).backward()
    b = logits.clone().requires_grad_(True)
    (oracle.switch_aux_loss(b, idx) * 2.0).backward()
    torch.testing.assert_close(a.grad.cpu(), b.grad, rtol=1e-4, atol=1e-8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["scatter2group", "group2scatter", "scatter2scatter", "group2group"])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("T,E,k,K,N", [(40, 4, 2, 64, 48), (300, 6, 3, 256, 264)])
def test_scattered_experts_is_differentiable(device, dtype, mode, gated, T, E, k, K, N):
    """ops.scattered_experts with tensors that require grad: value and gradients (inputs, expert weights, gates)
    against autograd through the oracle's fp32 restatement of the call."""
    from oracle import moe_oracle as oracle

    grouped_in, grouped_out = mode.startswith("group"), mode.endswith("group")
    if gated and grouped_out:
        pytest.skip("gates contract the flat-slot order")
    g = torch.Generator().manual_seed(T + K + N)
    sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    se, ss, off = oracle.sort_bin(sel, E)
    L = T * k
    x0 = torch.randn(L if grouped_in else T, K, generator=g).to(dtype)
    w0 = (torch.randn(E, N, K, generator=g) * 0.1).to(dtype)        # native (E, out, in)
    g0 = torch.rand(T, k, generator=g).to(dtype) if gated else None
    up = torch.randn(T if gated else L, N, generator=g).to(dtype)

    xr, wr = x0.float().clone().requires_grad_(True), w0.float().clone().requires_grad_(True)
    gr = g0.float().clone().requires_grad_(True) if gated else None
    ref = oracle.scattered_experts_oracle(xr, wr, k, se, ss, off, gates=gr, grouped_in=grouped_in, grouped_out=grouped_out)
    (ref * up.float()).sum().backward()

    ops = _ops()
    xd, wd = x0.to(device).requires_grad_(True), w0.to(device).requires_grad_(True)
    gd = g0.to(device).requires_grad_(True) if gated else None
    out = ops.scattered_experts(xd, wd.permute(0, 2, 1), k, se.to(device), ss.to(device), off.to(device), gates=gd,
                                grouped_in=grouped_in, grouped_out=grouped_out)
    (out * up.to(device)).sum().backward()

    tol = dict(rtol=2e-3, atol=2e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    torch.testing.assert_close(out.detach().cpu().float(), ref.detach(), **tol)
    for name, got, want in (("x", xd.grad, xr.grad), ("w", wd.grad, wr.grad)) + ((("gates", gd.grad, gr.grad),) if gated else ()):
        scale = want.abs().max().clamp_min(1e-6)
        torch.testing.assert_close(got.cpu().float() / scale, want / scale, rtol=tol["rtol"], atol=tol["rtol"]), name


def test_grouped_wgrad_full_size(device):
    """Granite-3B-A800M-shape weight gradients (262144 sorted rows, 40 experts, Zipf-like sizes, both uses of the
    kernel): every expert's block against a float32 product of the same rows computed by torch on the GPU, and the
    sum over experts against one dense product (a checksum that every row was used exactly once)."""
    ops = _ops()
    g = torch.Generator().manual_seed(11)
    T, k, E, H, I = 32768, 8, 40, 1536, 512
    L = T * k
    w = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.1
    counts = _seeded_counts(L, w, g)
    counts = counts[torch.randperm(E, generator=g)]
    offsets = counts.cumsum(0).to(torch.int32).to(device)
    tok = torch.randint(0, T, (L,), generator=g, dtype=torch.int32).to(device)
    d_h = (torch.randn(L, 2 * I, generator=g) * 0.5).to(torch.bfloat16).to(device)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(device)

    dw = ops.grouped_wgrad(d_h, x, offsets, None, tok)            # d c_fc: (E, 2I, H)
    assert tuple(dw.shape) == (E, 2 * I, H)
    xg = x[tok.long()]
    dense = d_h.float().t() @ xg.float()
    torch.testing.assert_close(dw.float().sum(0), dense, rtol=2e-2, atol=2e-2 * dense.abs().max().item())
    start = 0
    for e, end in enumerate(offsets.tolist()):
        if e % 7 == 0 or counts[e] == counts.max():
            ref = d_h[start:end].float().t() @ xg[start:end].float()
            torch.testing.assert_close(dw[e].float(), ref, rtol=2e-2, atol=1e-2 * ref.abs().max().item())
        start = end

    dy = torch.randn(T, H, generator=g).to(torch.bfloat16).to(device)
    act = (torch.randn(L, I, generator=g) * 0.5).to(torch.bfloat16).to(device)
    dp = ops.grouped_wgrad(dy, act, offsets, tok, None)           # d c_proj: (E, H, I)
    dense = dy[tok.long()].float().t() @ act.float()
    torch.testing.assert_close(dp.float().sum(0), dense, rtol=2e-2, atol=2e-2 * dense.abs().max().item())


@pytest.mark.parametrize("seed", list(range(12)))
def test_grouped_wgrad_random_shapes(device, seed):
    """Random shapes around the kernel's boundaries: row counts that straddle the group size, operand widths that
    leave partial 256-column tiles or more than 8 row tiles (several bands), many experts."""
    import random

    rnd = random.Random(seed)
    E = rnd.choice([1, 2, 7, 33, 64, 200, 256])
    L = rnd.choice([1, 31, 255, 257, 1000, 4097, 9001])
    M = 8 * rnd.choice([1, 5, 32, 33, 40, 260, 300])
    N = 8 * rnd.choice([1, 3, 31, 32, 65])
    g = torch.Generator().manual_seed(seed)
    counts = _seeded_counts(L, torch.rand(E, generator=g).pow(4) + 1e-6, g)
    offsets = counts.cumsum(0).to(torch.int32)
    rows_other = rnd.choice([1, 17, L])
    a = torch.randn(L, M, generator=g).to(torch.bfloat16)
    b = torch.randn(rows_other, N, generator=g).to(torch.bfloat16)
    b_idx = torch.randint(0, rows_other, (L,), generator=g, dtype=torch.int32)
    got = _ops().grouped_wgrad(a.to(device), b.to(device), offsets.to(device), None, b_idx.to(device))
    ref = _wgrad_reference(a, b, offsets, None, b_idx)
    torch.testing.assert_close(got.cpu().double(), ref, rtol=2.0 ** -7, atol=2e-5 * max(1.0, counts.max().item()) ** 0.5 + 1e-6)


@pytest.mark.parametrize("dtype,T,H,E,k", [(torch.bfloat16, 300, 128, 40, 8), (torch.float16, 257, 64, 136, 12),
                                           (torch.float32, 100, 64, 8, 2), (torch.bfloat16, 2100, 1536, 40, 8)])
def test_fused_router_function(device, dtype, T, H, E, k):
    """autograd.FusedRouter (router kernel forward; d-logits kernel + grouped GEMM + grouped weight gradient
    backward) against torch autograd through linear -> gather at the same experts -> float softmax -> cast
    (moe.py:246-257), with gradients arriving at the gates and at the logits."""
    from dolomite_engine_amd.autograd import FusedRouter

    g = torch.Generator().manual_seed(T + E)
    x0 = torch.randn(T, H, generator=g).to(dtype).to(device)
    w0 = (torch.randn(E, H, generator=g) * 0.1).to(dtype).to(device)
    dg = torch.randn(T, k, generator=g).to(dtype).to(device)
    dl = (torch.randn(T, E, generator=g) * 0.05).to(dtype).to(device)
    print(f"FusedRouter {dtype} T={T} H={H} E={E} k={k}", flush=True)

    x, w = x0.clone().requires_grad_(True), w0.clone().requires_grad_(True)
    logits, gates, experts, *srt = FusedRouter.apply(x, w, None, k)
    ((gates * dg).sum() + (logits * dl).sum()).backward()
    from dolomite_engine_amd import ops

    # where the router kernel folds the expert sort in, the function hands it back: the sort of its selection
    assert (srt[0] is not None) == ops.router_fused_sort_supported(x0, E, k)
    if srt[0] is not None:
        for got, want in zip(srt, ops.sort_bin(experts, E)):
            assert torch.equal(got, want)

    xr, wr = x0.clone().requires_grad_(True), w0.clone().requires_grad_(True)
    logits_r = torch.nn.functional.linear(xr, wr)
    gates_r = torch.softmax(logits_r.gather(-1, experts.long()).float(), dim=-1).to(dtype)
    ((gates_r * dg).sum() + (logits_r * dl).sum()).backward()

    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(logits.detach().float(), logits_r.detach().float(), **tol)
    for name, got, want in (("dx", x.grad, xr.grad), ("dw", w.grad, wr.grad)):
        scale = want.float().abs().max().clamp_min(1e-6)
        assert_close_scaled(got, want, dtype, what=f"router {name}", rtol=tol["rtol"], atol=tol["atol"] * scale.item(),
                            rel_to_max=2e-2 if dtype != torch.float32 else 1e-4,
                            rel_rms_limit=1e-2 if dtype != torch.float32 else 1e-4)
