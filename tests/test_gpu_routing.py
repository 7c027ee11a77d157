"""GPU parity of the routing kernels against the CPU oracle (bit-exact indices, counts, order)."""

import pytest
import torch

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


def _ops():
    from dolomite_engine_amd import ops

    return ops


def _logits(T, E, dtype, seed, ties=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, E, generator=g) * 0.7
    if ties:  # coarse grid: many exact ties, including at the k / k+1 boundary
        x = torch.round(x * 2) / 2
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k", [(1, 8, 2), (15, 8, 8), (512, 8, 2), (1000, 32, 8), (777, 40, 8), (64, 64, 6),
                                   (33, 5, 1), (129, 100, 7), (65, 256, 9), (31, 1000, 64), (16, 1, 1)])
@pytest.mark.parametrize("ties", [False, True])
def test_topk_softmax(device, dtype, T, E, k, ties):
    ops = _ops()
    logits = _logits(T, E, dtype, seed=T * 131 + E * 7 + k, ties=ties)
    print(f"topk T={T} E={E} k={k} {dtype} ties={ties}", flush=True)
    gates, idx = ops.router_topk_softmax(logits.to(device), k)
    vals, ref_idx = oracle.topk_canonical(logits, k)
    ref_gates = oracle.softmax_topk(vals, dtype)
    assert idx.dtype == torch.int32
    assert torch.equal(idx.cpu().long(), ref_idx), "expert indices differ from the canonical top-k"
    tol = {torch.float32: 2e-6, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
    torch.testing.assert_close(gates.cpu().float(), ref_gates.float(), rtol=tol, atol=tol * 0.1)
    # at most one unit in the last place anywhere
    if dtype != torch.float32:
        ulp_diff = (gates.cpu().view(torch.int16).int() - ref_gates.view(torch.int16).int()).abs().max()
        assert ulp_diff <= 1


def test_topk_special_values(device):
    ops = _ops()
    x = torch.tensor([[0.0, -0.0, 1.0, float("-inf"), 1.0, float("inf"), -2.0, 0.5],
                      [float("nan"), 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0]])
    gates, idx = ops.router_topk_softmax(x.to(device), 4)
    assert idx[0].tolist() == [5, 2, 4, 7]
    assert idx[1].tolist()[0] == 0  # NaN orders first, as in torch
    _, ref = oracle.topk_canonical(x, 4)
    assert torch.equal(idx.cpu().long(), ref)
    # -0.0 and +0.0 tie: lower index first
    y = torch.tensor([[-0.0, 0.0, -1.0, -1.0]])
    _, idx = ops.router_topk_softmax(y.to(device), 2)
    assert idx[0].tolist() == [0, 1]


@pytest.mark.parametrize("T,k,E", [(0, 2, 8), (1, 1, 1), (15, 8, 8), (512, 2, 8), (64, 6, 64), (1024, 8, 32),
                                   (1365, 6, 40), (16384, 8, 32), (32768, 8, 40), (5000, 3, 1000), (4099, 2, 3),
                                   (70000, 8, 40)])  # the last: more chunks than the launch that fuses passes 2 and 3 takes
@pytest.mark.parametrize("skew", [False, True])
def test_sort_bin(device, T, k, E, skew):
    ops = _ops()
    g = torch.Generator().manual_seed(T + 17 * k + E)
    if skew:
        p = torch.arange(1, E + 1, dtype=torch.float64).pow(-1.1)
        sel = torch.multinomial(p.expand(max(T, 1), E), min(k, E), replacement=False, generator=g)[:T]
        if k > E:
            pytest.skip("k > E")
    else:
        sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    sel = sel.reshape(T, k)
    print(f"sort_bin T={T} k={k} E={E} skew={skew}", flush=True)
    se, ss, off = ops.sort_bin(sel.to(device=device, dtype=torch.int32), E)
    rse, rss, roff = oracle.sort_bin(sel, E)
    assert torch.equal(off.cpu().long(), roff)
    assert torch.equal(se.cpu().long(), rse)
    assert torch.equal(ss.cpu().long(), rss)


def test_sort_bin_all_one_expert(device):
    ops = _ops()
    T, k, E = 9000, 1, 16
    sel = torch.full((T, k), 11, dtype=torch.int32)
    se, ss, off = ops.sort_bin(sel.to(device), E)
    assert torch.equal(ss.cpu().long(), torch.arange(T))
    assert off.cpu().tolist() == [0] * 11 + [T] * 5
    assert bool((se == 11).all())


@pytest.mark.parametrize("L,E", [(0, 4), (1, 1), (1000, 8), (262144, 40), (100003, 1000)])
def test_count(device, L, E):
    ops = _ops()
    g = torch.Generator().manual_seed(L + E)
    ids = torch.randint(0, E, (L,), generator=g)
    got = ops.continuous_count(ids.to(device), E)
    assert got.dtype == torch.uint32
    assert torch.equal(got.cpu().to(torch.int64), torch.bincount(ids, minlength=E))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,k,bias", [(1, 64, 8, 2, False), (15, 32, 8, 8, False), (200, 256, 40, 8, True),
                                          (1000, 1024, 32, 8, False), (64, 4096, 64, 6, False),
                                          (333, 1536, 40, 8, True), (130, 48, 5, 1, False),
                                          (2500, 256, 40, 8, True), (4099, 512, 64, 6, False),
                                          # many tokens, gate weights beyond LDS: K split across a workgroup's waves
                                          (1500, 4096, 64, 6, True), (2049, 2064, 50, 8, False),
                                          (1090, 5008, 17, 3, True)])
def test_router_fused(device, dtype, T, H, E, k, bias):
    ops = _ops()
    g = torch.Generator().manual_seed(T + H + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    w = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    b = (torch.randn(E, generator=g) * 0.5) if bias else None
    print(f"router_fused T={T} H={H} E={E} k={k} {dtype} bias={bias}", flush=True)
    logits, gates, idx = ops.router_fused(x.to(device), w.to(device), k, bias=None if b is None else b.to(device),
                                          return_logits=True)
    logits = logits.cpu()
    # (1) the logits are the oracle's up to one rounding step of the model dtype
    ref_logits = oracle.router_logits(x, w, b)
    # (with a bias the product is rounded before the bias is added: where the two cancel, one rounding step of the
    # product is large against the sum)
    atol = 1e-3
    if b is not None:
        atol += (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11) * float((ref_logits.float() - b).abs().max())
    torch.testing.assert_close(logits.float(), ref_logits.float(), rtol=1.6e-2 if dtype == torch.bfloat16 else 2e-3,
                               atol=atol)
    # (2) given the device's own logits, routing is bit-exact
    vals, ref_idx = oracle.topk_canonical(logits, k)
    assert torch.equal(idx.cpu().long(), ref_idx)
    ref_gates = oracle.softmax_topk(vals, dtype)
    ulp = (gates.cpu().view(torch.int16).int() - ref_gates.view(torch.int16).int()).abs().max()
    assert ulp <= 1
    # (3) without materialising the logits the result is the same
    _, gates2, idx2 = ops.router_fused(x.to(device), w.to(device), k, bias=None if b is None else b.to(device))
    assert torch.equal(idx2, idx) and torch.equal(gates2, gates)
    # (4) the single-launch kernel (no workspace) sums K in another order: same contract on its own logits
    logits3, gates3, idx3 = ops.router_fused(x.to(device), w.to(device), k, bias=None if b is None else b.to(device),
                                             return_logits=True, split_k=False)
    torch.testing.assert_close(logits3.cpu().float(), ref_logits.float(),
                               rtol=1.6e-2 if dtype == torch.bfloat16 else 2e-3, atol=atol)
    vals3, ref_idx3 = oracle.topk_canonical(logits3.cpu(), k)
    assert torch.equal(idx3.cpu().long(), ref_idx3)
    ulp3 = (gates3.cpu().view(torch.int16).int() - oracle.softmax_topk(vals3, dtype).view(torch.int16).int()).abs().max()
    assert ulp3 <= 1


@pytest.mark.parametrize("dtype,T,H,E,k,bias", [
    (torch.float32, 512, 256, 8, 2, False),      # the reference's correctness configuration
    (torch.float32, 1, 8, 4, 1, False),
    (torch.float32, 333, 136, 40, 8, True),
    (torch.float32, 70, 1536, 200, 33, True),
    (torch.bfloat16, 300, 256, 128, 8, True),    # more than 64 experts
    (torch.float16, 129, 1024, 256, 64, False),  # k beyond the streaming kernels' 8
    (torch.bfloat16, 50, 64, 40, 12, False),
    (torch.bfloat16, 2100, 48, 65, 2, False),
    # many tokens, more than 64 experts, 16-bit: logits from the grouped GEMM's tile kernels, then the top-k kernel
    (torch.bfloat16, 8200, 256, 128, 8, False),
    (torch.float16, 4100, 512, 256, 6, False),
    (torch.bfloat16, 10500, 48, 100, 20, False),   # (100 experts, hidden 48: not every tile kernel's shape)
    (torch.bfloat16, 8200, 256, 128, 8, True),     # with a bias: the general kernel
    # few tokens, more than 64 experts: the contraction cut into ranges over many workgroups
    (torch.bfloat16, 64, 7168, 256, 8, False),
    (torch.float16, 1, 2048, 128, 8, True),
    (torch.bfloat16, 1000, 2064, 200, 20, True),
    (torch.float32, 33, 4096, 130, 6, False),
])
def test_router_general(device, dtype, T, H, E, k, bias):
    """fp32, more than 64 experts, k above 8: the general kernel behind the same entry point, held to the same
    contract as the streaming kernels (logits = the oracle's up to the summation order, routing bit-exact on the
    device's own logits, gates within one unit in the last place)."""
    ops = _ops()
    g = torch.Generator().manual_seed(T + H + E + k)
    x = torch.randn(T, H, generator=g).to(dtype)
    w = (torch.randn(E, H, generator=g) * 0.05).to(dtype)
    b = (torch.randn(E, generator=g) * 0.5) if bias else None
    print(f"router general T={T} H={H} E={E} k={k} {dtype} bias={bias}", flush=True)
    assert ops.router_fused_supported(x, E, k)
    bd = None if b is None else b.to(device)
    logits, gates, idx = ops.router_fused(x.to(device), w.to(device), k, bias=bd, return_logits=True)
    logits = logits.cpu()
    ref_logits = oracle.router_logits(x, w, b)
    tol = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=1.6e-2, atol=1e-3),
           torch.float16: dict(rtol=2e-3, atol=1e-3)}[dtype]
    if b is not None and dtype != torch.float32:
        # (the product is rounded before the bias is added: where the two cancel, one rounding step of the product
        # is large against the sum)
        tol["atol"] += (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11) * float((ref_logits.float() - b).abs().max())
    torch.testing.assert_close(logits.float(), ref_logits.float(), **tol)
    vals, ref_idx = oracle.topk_canonical(logits, k)
    assert torch.equal(idx.cpu().long(), ref_idx)
    ref_gates = oracle.softmax_topk(vals, dtype)
    if dtype == torch.float32:
        torch.testing.assert_close(gates.cpu(), ref_gates, rtol=1e-5, atol=1e-7)
    else:
        assert (gates.cpu().view(torch.int16).int() - ref_gates.view(torch.int16).int()).abs().max() <= 1
    _, gates2, idx2 = ops.router_fused(x.to(device), w.to(device), k, bias=bd)
    assert torch.equal(idx2, idx) and torch.equal(gates2, gates)
    # without a workspace (one launch; few tokens with many experts, and many tokens, take other forms with one):
    # another summation order, the same contract on its own logits
    logits3, gates3, idx3 = ops.router_fused(x.to(device), w.to(device), k, bias=bd, return_logits=True, split_k=False)
    torch.testing.assert_close(logits3.cpu().float(), ref_logits.float(), **tol)
    vals3, ref_idx3 = oracle.topk_canonical(logits3.cpu(), k)
    assert torch.equal(idx3.cpu().long(), ref_idx3)
    ref_gates3 = oracle.softmax_topk(vals3, dtype)
    if dtype == torch.float32:
        torch.testing.assert_close(gates3.cpu(), ref_gates3, rtol=1e-5, atol=1e-7)
    else:
        assert (gates3.cpu().view(torch.int16).int() - ref_gates3.view(torch.int16).int()).abs().max() <= 1


def test_router_general_ties_and_special_values(device):
    """Tie rule of the general kernel on logits built to tie: equal columns in the gate weight give equal logits
    for every token; the lower expert index must win."""
    ops = _ops()
    T, H, E, k = 40, 64, 130, 5
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    base = (torch.randn(7, H, generator=g) * 0.1).to(torch.bfloat16)
    w = base[torch.arange(E) % 7].contiguous()          # 130 experts, only 7 distinct rows: ties everywhere
    logits, gates, idx = ops.router_fused(x.to(device), w.to(device), k, return_logits=True)
    vals, ref_idx = oracle.topk_canonical(logits.cpu(), k)
    assert torch.equal(idx.cpu().long(), ref_idx)
    assert (gates.cpu().view(torch.int16).int() - oracle.softmax_topk(vals, torch.bfloat16).view(torch.int16).int()).abs().max() <= 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k", [(1, 4, 1), (15, 8, 8), (300, 40, 8), (129, 130, 2), (70, 256, 64)])
@pytest.mark.parametrize("parts", ["gates", "extra", "both"])
def test_router_dlogits(device, dtype, T, E, k, parts):
    """d logits from (d gates, d logits_extra) against torch autograd through gather -> float softmax -> cast
    (moe.py:250-255), in fp32 and rounded where autograd rounds."""
    ops = _ops()
    g = torch.Generator().manual_seed(T * 7 + E + k)
    logits = torch.randn(T, E, generator=g).to(dtype)
    _, idx = oracle.topk_canonical(logits, k)
    d_gates = torch.randn(T, k, generator=g).to(dtype) if parts != "extra" else None
    extra = (torch.randn(T, E, generator=g) * 0.1).to(dtype) if parts != "gates" else None
    got = ops.router_dlogits(logits.to(device), idx.to(torch.int32).to(device),
                             None if d_gates is None else d_gates.to(device),
                             None if extra is None else extra.to(device)).cpu()
    lg = logits.clone().requires_grad_(True)
    want = torch.zeros(T, E, dtype=dtype)
    if d_gates is not None:
        gates = torch.softmax(lg.gather(-1, idx).float(), dim=-1).to(dtype)
        (gates * d_gates).sum().backward()
        want = lg.grad
    if extra is not None:
        want = want + extra
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=0, atol=0)
    if dtype != torch.float32:
        # same fp32 arithmetic up to the order of the softmax's sum: a unit in the last place here and there
        steps = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
        close = (got.float() - want.float()).abs() <= 1e-3 * want.float().abs() + 2e-6
        assert bool(((steps <= 1) | close).all())
    else:
        torch.testing.assert_close(got, want, **tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,k,bias,gamma", [(1, 64, 8, 2, False, True), (200, 256, 40, 8, True, True),
                                                (2500, 1536, 40, 8, True, True), (4099, 1024, 32, 8, False, False),
                                                (333, 48, 5, 1, False, True)])
def test_rmsnorm_router_fused(device, dtype, T, H, E, k, bias, gamma):
    """RMSNorm folded into the router kernel: x_norm equals the oracle's RMSNorm up to one unit in the last place
    (the sum of squares is added in another order), and everything after it is the fused router's contract on the
    device's own x_norm."""
    ops = _ops()
    g = torch.Generator().manual_seed(T + H + E)
    h = (torch.randn(T, H, generator=g) * 2.5).to(dtype)
    lnw = (1 + 0.2 * torch.randn(H, generator=g)).to(dtype) if gamma else None
    w = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    b = (torch.randn(E, generator=g) * 0.5) if bias else None
    assert ops.rmsnorm_router_fused_supported(h.to(device), E, k)
    print(f"rmsnorm_router_fused T={T} H={H} E={E} k={k} {dtype}", flush=True)
    x_norm, logits, gates, idx = ops.rmsnorm_router_fused(
        h.to(device), None if lnw is None else lnw.to(device), 1e-5, w.to(device), k,
        bias=None if b is None else b.to(device), return_logits=True)
    ref_norm = oracle.rmsnorm(h, lnw, 1e-5)
    bits = torch.int16
    ulp = (x_norm.cpu().view(bits).int() - ref_norm.view(bits).int()).abs()
    assert ulp.max() <= 1 and (ulp > 0).float().mean() < 1e-3
    # from here on: the fused router on the device's x_norm
    xn = x_norm.cpu()
    ref_logits = oracle.router_logits(xn, w, b)
    torch.testing.assert_close(logits.cpu().float(), ref_logits.float(), rtol=1.6e-2 if dtype == torch.bfloat16 else 2e-3,
                               atol=1e-3)
    vals, ref_idx = oracle.topk_canonical(logits.cpu(), k)
    assert torch.equal(idx.cpu().long(), ref_idx)
    ref_gates = oracle.softmax_topk(vals, dtype)
    assert (gates.cpu().view(bits).int() - ref_gates.view(bits).int()).abs().max() <= 1
    # and the unfused pair of calls on that x_norm gives the same routing
    logits2, gates2, idx2 = ops.router_fused(x_norm, w.to(device), k, bias=None if b is None else b.to(device),
                                             return_logits=True)
    torch.testing.assert_close(logits2.float(), logits.float(), rtol=1.6e-2 if dtype == torch.bfloat16 else 2e-3, atol=1e-3)


def test_rmsnorm_router_fused_unsupported_shapes(device):
    ops = _ops()
    x = torch.zeros(4, 4096, dtype=torch.bfloat16, device=device)
    assert not ops.rmsnorm_router_fused_supported(x, 64, 6)       # 64 x 4096 gate weights do not fit in LDS
    assert ops.rmsnorm_router_fused_supported(x, 8, 2)
    assert not ops.rmsnorm_router_fused_supported(x.float(), 8, 2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,k,bias", [(1, 64, 8, 2, False), (15, 32, 8, 8, False), (64, 4096, 64, 6, False),
                                          (200, 256, 40, 8, True), (1000, 1024, 32, 8, False), (1024, 512, 64, 8, True),
                                          (130, 48, 5, 1, False), (320, 1536, 40, 8, True), (1024, 4096, 64, 6, False),
                                          # just past the few-token form where the gate weights fit in LDS
                                          (321, 1536, 40, 8, True), (768, 1024, 32, 8, False),
                                          # many tokens: the router counts the experts per chunk for the sort
                                          (1025, 64, 8, 2, False), (2500, 256, 40, 8, True), (4099, 512, 64, 6, False),
                                          (16384, 1024, 32, 8, False), (32768, 1536, 40, 8, True),
                                          (70001, 128, 40, 1, False), (40000, 256, 16, 3, True)])
def test_router_fused_sort_equals_separate_calls(device, dtype, T, H, E, k, bias):
    """The router call that also sorts -- few tokens: its finishing launch sorts; many tokens: its epilogue counts
    the experts per chunk and the sort's scan and scatter passes follow -- must give exactly what the fused router
    followed by mi_moe_sort_bin gives (logits, gates, experts, sorted order, offsets), and the sort must be the
    oracle's.  Called twice, so that a counter left over from the first call would show."""
    ops = _ops()
    g = torch.Generator().manual_seed(T * 7 + H + E)
    x = torch.randn(T, H, generator=g).to(dtype).to(device)
    w = (torch.randn(E, H, generator=g) * 0.05).to(dtype).to(device)
    b = torch.randn(E, generator=g).to(device) if bias else None
    assert ops.router_fused_sort_supported(x, E, k)
    print(f"router_fused_sort T={T} H={H} E={E} k={k} bias={bias} {dtype}", flush=True)
    ref_logits, ref_gates, ref_idx = ops.router_fused(x, w, k, bias=b, return_logits=True)
    ref_se, ref_ss, ref_off = ops.sort_bin(ref_idx, E)
    for _ in range(2):
        logits, gates, idx, se, ss, off = ops.router_fused_sort(x, w, k, bias=b, return_logits=True)
        torch.cuda.synchronize()
        assert torch.equal(logits, ref_logits) and torch.equal(gates, ref_gates) and torch.equal(idx, ref_idx)
        assert torch.equal(se, ref_se) and torch.equal(ss, ref_ss) and torch.equal(off, ref_off)
    ose, oss, ooff = oracle.sort_bin(ref_idx.cpu().long(), E)
    assert torch.equal(se.cpu().long(), ose) and torch.equal(ss.cpu().long(), oss) and torch.equal(off.cpu().long(), ooff)


def test_router_fused_sort_limits(device):
    ops = _ops()
    x = torch.zeros(2048, 64, dtype=torch.bfloat16, device=device)
    assert ops.router_fused_sort_supported(x, 8, 2)              # many tokens: the form that counts per chunk
    assert not ops.router_fused_sort_supported(torch.zeros(2048, 4096, dtype=torch.bfloat16, device=device), 64, 2)  # gate weights beyond LDS
    assert not ops.router_fused_sort_supported(x[:1024], 64, 9)  # k beyond the fused router
    assert ops.router_fused_sort_supported(x[:1024], 64, 8)      # 8192 slots: the one-block sort's limit
    big = torch.zeros(1025, 4096, dtype=torch.bfloat16, device=device)
    assert ops.router_fused_sort_supported(big[:1024], 64, 6)    # gate weights beyond LDS: the few-token form up to 1024
    assert not ops.router_fused_sort_supported(big, 64, 6)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_routing_random_shapes(device, seed):
    """Random shapes through every form of the routing stage -- streaming router, general router (fp32, many
    experts, large k), router + sort in both its forms, stand-alone sort -- against the oracle: routing bit-exact on
    the device's own logits, sort bit-exact, and the fused forms bit-identical to the separate calls."""
    import random

    ops = _ops()
    rnd = random.Random(seed)
    for case in range(24):
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        E = rnd.choice([1, 2, 5, 8, 16, 40, 64, 65, 100, 128, 200, 256])
        k = min(rnd.choice([1, 2, 3, 6, 8, 9, 20]), E)
        T = rnd.choice([1, 3, 16, 17, 100, 512, 1024, 1025, 1500, 4099, 9000])
        H = 16 * rnd.choice([1, 2, 3, 8, 17, 48, 64, 96])
        bias = rnd.choice([False, True])
        g = torch.Generator().manual_seed(seed * 7919 + case)
        x = torch.randn(T, H, generator=g).to(dtype)
        w = (torch.randn(E, H, generator=g) * 0.05).to(dtype)
        b = (torch.randn(E, generator=g) * 0.3) if bias else None
        print(f"routing random seed {seed} case {case}: T={T} H={H} E={E} k={k} {dtype} bias={bias}", flush=True)
        xd, wd, bd = x.to(device), w.to(device), None if b is None else b.to(device)
        assert ops.router_fused_supported(xd, E, k)
        logits, gates, idx = ops.router_fused(xd, wd, k, bias=bd, return_logits=True)
        ref_logits = oracle.router_logits(x, w, b)
        tol = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=1.6e-2, atol=2e-3),
               torch.float16: dict(rtol=2e-3, atol=1e-3)}[dtype]
        if b is not None and dtype != torch.float32:
            # the product is rounded before the bias is added: where the two cancel, one rounding step of the
            # product is large against the sum
            step = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
            tol["atol"] += step * float((ref_logits.float() - b).abs().max())
        torch.testing.assert_close(logits.cpu().float(), ref_logits.float(), **tol)
        vals, ref_idx = oracle.topk_canonical(logits.cpu(), k)
        assert torch.equal(idx.cpu().long(), ref_idx), case
        ref_gates = oracle.softmax_topk(vals, dtype)
        if dtype == torch.float32:
            torch.testing.assert_close(gates.cpu(), ref_gates, rtol=1e-5, atol=1e-7)
        else:
            assert (gates.cpu().view(torch.int16).int() - ref_gates.view(torch.int16).int()).abs().max() <= 1
        se, ss, off = ops.sort_bin(idx, E)
        ose, oss, ooff = oracle.sort_bin(ref_idx, E)
        assert torch.equal(se.cpu().long(), ose) and torch.equal(ss.cpu().long(), oss) and torch.equal(off.cpu().long(), ooff)
        if ops.router_fused_sort_supported(xd, E, k):
            l2, g2, i2, se2, ss2, off2 = ops.router_fused_sort(xd, wd, k, bias=bd, return_logits=True)
            assert torch.equal(l2, logits) and torch.equal(g2, gates) and torch.equal(i2, idx), case
            assert torch.equal(se2, se) and torch.equal(ss2, ss) and torch.equal(off2, off), case
        # backward of the routing: d logits for random incoming gradients against autograd
        d_gates = torch.randn(T, k, generator=g).to(dtype)
        got = ops.router_dlogits(logits, idx, d_gates.to(device), None).cpu()
        lg = logits.cpu().clone().requires_grad_(True)
        (torch.softmax(lg.gather(-1, ref_idx).float(), dim=-1).to(dtype) * d_gates).sum().backward()
        if dtype == torch.float32:
            torch.testing.assert_close(got, lg.grad, rtol=1e-4, atol=1e-6)
        else:
            steps = (got.view(torch.int16).int() - lg.grad.view(torch.int16).int()).abs()
            close = (got.float() - lg.grad.float()).abs() <= 1e-3 * lg.grad.float().abs() + 2e-6
            assert bool(((steps <= 1) | close).all()), case
