"""GPU parity of the grouped GEMM / SwiGLU / combine / fp8 kernels against the fp32 CPU oracle.

Tolerances: bf16 / fp16 results are compared with the fp32 oracle at rtol = atol = 2e-2 (the stated
acceptance bar); fp32 results at rtol 1e-3 / atol 2e-4 (the reference's own fp32 tolerance for this
path, tests/hf_models/single_gpu/scattermoe_test.py:38-48).
"""

import pytest
import torch

from oracle import moe_oracle as oracle

from _parity import assert_close_scaled

pytestmark = pytest.mark.gpu

TOL = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=2e-2, atol=2e-2),
       torch.float16: dict(rtol=2e-2, atol=2e-2)}


def _ops():
    from dolomite_engine_amd import ops

    return ops


def _routing(T, E, k, seed, skew=False):
    g = torch.Generator().manual_seed(seed)
    noise = torch.rand(T, E, generator=g)
    if skew:
        noise = noise + torch.arange(E, dtype=torch.float32).pow(1.2) * 0.05
    sel = noise.argsort(dim=1)[:, :k]
    return oracle.sort_bin(sel, E)


def _rand(shape, std, dtype, g):
    return (torch.randn(*shape, generator=g) * std).to(dtype)


CASES = [
    # T, E, k, K, N
    (15, 8, 8, 32, 128),
    (64, 8, 2, 64, 64),
    (300, 4, 2, 256, 512),
    (1, 4, 1, 64, 96),
    (257, 5, 3, 72, 100),     # K % 64 != 0, N % 32 != 0
    (1024, 8, 2, 256, 1024),
    (700, 3, 2, 128, 260),
    (5000, 6, 3, 160, 520),   # many tiles per workgroup-list, tails in rows and columns
    (3000, 130, 2, 128, 72),  # more than 64 experts (second chunk of the tile table), most of them nearly empty
    (700, 250, 1, 256, 264),  # many empty experts
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,E,k,K,N", CASES)
@pytest.mark.parametrize("mode", ["scatter2group", "group2scatter", "scatter2scatter", "group2group"])
@pytest.mark.parametrize("cfg", [-1, 0, 1, 2, 3, 4, 5, 7, 8, 9])
def test_scattered_gemm(device, dtype, T, E, k, K, N, mode, cfg):
    if dtype == torch.float32 and cfg in (4, 7, 8, 9):
        pytest.skip("the DMA-staged configurations are 16-bit only")
    if cfg == 4 and K % 32:
        pytest.skip("the DMA-staged kernel needs K % 32 == 0")
    if cfg in (7, 8, 9) and (K % 32 or K < 128 or N % 8):
        pytest.skip("the persistent kernel needs K % 32 == 0, K >= 128, N % 8 == 0")
    ops = _ops()
    g = torch.Generator().manual_seed(T * 3 + E + K + N)
    se, ss, off = _routing(T, E, k, seed=T + E, skew=(T % 2 == 0))
    L = T * k
    grouped_in = mode.startswith("group")
    grouped_out = mode.endswith("group")
    x = _rand((L if grouped_in else T, K), 1.0, dtype, g)
    w = _rand((E, N, K), 0.05, dtype, g)
    print(f"gemm {mode} cfg={cfg} T={T} E={E} k={k} K={K} N={N} {dtype}", flush=True)
    out = ops.scattered_gemm(x.to(device), w.to(device), k, ss.to(device), off.to(device), grouped_in, grouped_out, cfg=cfg)
    ref = oracle.scattered_experts_oracle(x, w, k, se, ss, off, grouped_in=grouped_in, grouped_out=grouped_out)
    torch.testing.assert_close(out.cpu().float(), ref, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,E,k,K,N", CASES + [(900, 4, 2, 1024, 1536), (2048, 8, 2, 512, 72)])
@pytest.mark.parametrize("mode", ["scatter2group", "group2scatter"])
def test_scattered_gemm_weight_kn(device, dtype, T, E, k, K, N, mode):
    """Weights stored (E, K, N), as both data gradients of the backward use them: against the oracle, and bit for
    bit against the native-layout kernel on a transposed copy where the transposed-weight kernel runs (same tile
    shape, same order of the contraction)."""
    ops = _ops()
    g = torch.Generator().manual_seed(T * 5 + E + K + N)
    se, ss, off = _routing(T, E, k, seed=T + E + 1, skew=(T % 2 == 0))
    L = T * k
    grouped_in = mode.startswith("group")
    grouped_out = mode.endswith("group")
    x = _rand((L if grouped_in else T, K), 1.0, dtype, g)
    w_kn = _rand((E, K, N), 0.05, dtype, g)
    print(f"gemm weight_kn {mode} T={T} E={E} k={k} K={K} N={N} {dtype}", flush=True)
    xd, wd, ssd, offd = x.to(device), w_kn.to(device), ss.to(device), off.to(device)
    out = ops.scattered_gemm(xd, wd, k, ssd, offd, grouped_in, grouped_out, weight_kn=True)
    ref = oracle.scattered_experts_oracle(x, w_kn.transpose(1, 2).contiguous(), k, se, ss, off, grouped_in=grouped_in,
                                          grouped_out=grouped_out)
    torch.testing.assert_close(out.cpu().float(), ref, **TOL[dtype])
    if dtype != torch.float32 and K % 32 == 0 and K >= 128 and N % 8 == 0:
        same = ops.scattered_gemm(xd, wd.transpose(1, 2).contiguous(), k, ssd, offd, grouped_in, grouped_out, cfg=7)
        assert torch.equal(out, same)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,E,k,H,I", [(15, 8, 8, 32, 128), (512, 8, 2, 256, 512), (333, 5, 2, 136, 100),
                                       (2048, 4, 2, 512, 256), (64, 64, 6, 256, 128)])
@pytest.mark.parametrize("cfg", [-1, 0, 1, 2, 3, 4, 5, 7, 8, 9])
def test_up_swiglu(device, dtype, T, E, k, H, I, cfg):
    if dtype == torch.float32 and cfg in (4, 7, 8, 9):
        pytest.skip("the DMA-staged configurations are 16-bit only")
    if cfg == 4 and H % 32:
        pytest.skip("the DMA-staged kernel needs K % 32 == 0")
    if cfg in (7, 8, 9) and (H % 32 or H < 128 or I % 8):
        pytest.skip("the persistent kernel needs K % 32 == 0, K >= 128, N % 8 == 0")
    ops = _ops()
    g = torch.Generator().manual_seed(T + H + I)
    se, ss, off = _routing(T, E, k, seed=T + 3 * E, skew=True)
    x = _rand((T, H), 1.0, dtype, g)
    w = _rand((E, 2 * I, H), 0.08, dtype, g)
    print(f"up_swiglu cfg={cfg} T={T} E={E} k={k} H={H} I={I} {dtype}", flush=True)
    act = ops.up_swiglu(x.to(device), w.to(device), k, ss.to(device), off.to(device), cfg=cfg)
    h = oracle.scattered_experts_oracle(x, w, k, se, ss, off, grouped_out=True)
    ref = oracle.swiglu(h)
    torch.testing.assert_close(act.cpu().float(), ref, **TOL[dtype])


def test_gemm_identity_weights_permutes_rows(device):
    """With identity expert weights the grouped GEMM is a pure gather / scatter: exact equality."""
    ops = _ops()
    T, E, k, K = 200, 6, 3, 64
    se, ss, off = _routing(T, E, k, seed=5)
    g = torch.Generator().manual_seed(1)
    x = _rand((T, K), 1.0, torch.bfloat16, g)
    w = torch.eye(K).expand(E, K, K).contiguous().to(torch.bfloat16)
    out = ops.scattered_gemm(x.to(device), w.to(device), k, ss.to(device), off.to(device), False, True)
    assert torch.equal(out.cpu(), x[ss // k])
    out2 = ops.scattered_gemm(out, w.to(device), 1, ss.to(device), off.to(device), True, False)
    assert torch.equal(out2.cpu(), x.repeat_interleave(k, dim=0))


@pytest.mark.parametrize("cfg", [2, 3, 4, 5, 7, 9])
def test_gemm_bf16_rounding_is_nearest_even(device, cfg):
    """The final fp32 -> bf16 rounding is round-to-nearest-even, bit for bit (ties, carries into the
    exponent, overflow to inf, NaN): out = a + b where the fp32 sum is exact, so the only rounding in the
    whole computation is the conversion of the result.  (fp32-denormal results are left out: what the
    matrix cores do with denormal operands is not part of the contract.)"""
    ops = _ops()
    g = torch.Generator().manual_seed(11)
    T, K, N = 8192, 128, 8
    # a: random normal bf16 bit patterns with moderate exponents, b: a few binades (0..12) below a
    a_bits = (torch.randint(0, 2, (T,), generator=g) << 15) | (torch.randint(100, 150, (T,), generator=g) << 7) \
        | torch.randint(0, 128, (T,), generator=g)
    shift = torch.randint(0, 13, (T,), generator=g)
    b_bits = (torch.randint(0, 2, (T,), generator=g) << 15) | ((((a_bits >> 7) & 0xff) - shift) << 7) \
        | torch.randint(0, 128, (T,), generator=g)
    a = a_bits.to(torch.int16).view(torch.bfloat16)
    b = b_bits.to(torch.int16).view(torch.bfloat16)
    # hand-made rows: exact ties (to even, both directions), carry into the next binade, overflow, NaN, inf
    special = [(1.0, 2.0 ** -8), (1.0 + 2.0 ** -7, 2.0 ** -8), (1.0, 2.0 ** -8 + 2.0 ** -15), (1.9921875, 2.0 ** -8),
               (-1.0, -(2.0 ** -8)), (3.3895313892515355e38, 3.3895313892515355e38), (float("nan"), 1.0),
               (float("inf"), 1.0), (float("-inf"), 1.0), (0.0, 0.0), (1.0, -1.0)]
    for i, (u, v) in enumerate(special):
        a[i], b[i] = u, v
    x = torch.zeros(T, K, dtype=torch.bfloat16)
    x[:, 0], x[:, 77] = a, b
    w = torch.zeros(1, N, K, dtype=torch.bfloat16)
    w[0, :, 0] = 1.0
    w[0, :, 77] = 1.0
    idx = torch.arange(T, dtype=torch.int32)
    off = torch.tensor([T], dtype=torch.int32)
    out = ops.scattered_gemm(x.to(device), w.to(device), 1, idx.to(device), off.to(device), False, False, cfg=cfg).cpu()
    want = (a.float() + b.float()).to(torch.bfloat16)
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(out[:, 0]), nan)
    for n in range(N):
        assert torch.equal(out[~nan, n].view(torch.int16), want[~nan].view(torch.int16)), n


def test_gemm_empty_experts_and_single_expert(device):
    ops = _ops()
    g = torch.Generator().manual_seed(3)
    T, E, k, K, N = 500, 16, 1, 128, 64
    sel = torch.full((T, 1), 9)  # every token to expert 9, the other 15 are empty
    se, ss, off = oracle.sort_bin(sel, E)
    x = _rand((T, K), 1.0, torch.bfloat16, g)
    w = _rand((E, N, K), 0.05, torch.bfloat16, g)
    for cfg in (0, 1, 2, 3, 4, 5, 7, 8, 9):
        out = ops.scattered_gemm(x.to(device), w.to(device), k, ss.to(device), off.to(device), False, False, cfg=cfg)
        ref = x.float() @ w[9].float().t()
        torch.testing.assert_close(out.cpu().float(), ref, rtol=2e-2, atol=2e-2)


# Shapes whose last round of 256 x 256 tiles is partly filled and whose contraction is long enough for the persistent
# kernel to cut those tiles along K (with 256 CUs: four parts per tile, two parts per tile, one tile per XCD, and
# the chip-wide last round of the interleaved tile order).
SPLIT_K_CASES = [
    ("four parts", [5000, 5000, 5000, 5000], 8192, 1024),
    ("two parts", [7000, 6000, 5200, 5000], 8192, 1024),
    ("ragged", [1, 9000, 0, 300, 12000, 257], 6144, 768),
    ("eight column tiles", [3000, 2500, 2000, 1500], 8192, 2048),  # the tile order that interleaves the XCDs
]


@pytest.mark.parametrize("form", ["plain", "swiglu", "weight_kn"])
@pytest.mark.parametrize("name,counts,K,N", SPLIT_K_CASES)
def test_split_k_of_the_last_round(device, form, name, counts, K, N):
    """The persistent kernel with its workspace (tiles of the last round cut along K, summed by the finishing
    launch) against the same kernel without it and against an fp32 product of the same rounded operands:
    same results up to the order of the fp32 sums, and the same bits from run to run."""
    ops = _ops()
    g = torch.Generator().manual_seed(len(counts) * 131 + K)
    E, L = len(counts), sum(counts)
    off = torch.tensor(counts).cumsum(0).to(torch.int32).to(device)
    ss = torch.randperm(L, generator=g).to(torch.int32).to(device)     # scattered output rows
    inp = (torch.randn(L, K, generator=g) * 0.5).to(torch.bfloat16).to(device)
    rows_w = 2 * N if form == "swiglu" else N
    w = (torch.randn(E, rows_w, K, generator=g) * 0.05).to(torch.bfloat16).to(device)
    w_kn = w.transpose(1, 2).contiguous() if form == "weight_kn" else None
    print(f"split-K {form} {name}", flush=True)

    def run(split):
        if form == "swiglu":
            return ops.up_swiglu(inp, w, 1, torch.arange(L, dtype=torch.int32, device=device), off, cfg=7, split_k=split)
        if form == "weight_kn":
            return ops.scattered_gemm(inp, w_kn, 1, ss, off, True, False, weight_kn=True, split_k=split)
        return ops.scattered_gemm(inp, w, 1, ss, off, True, False, cfg=7, split_k=split)

    whole, split, again = run(False), run(True), run(True)
    assert torch.equal(split, again), "not reproducible"
    # fp32 product of the same operands, expert by expert (a library GEMM on the device)
    ref = torch.empty((L, N), dtype=torch.float32, device=device)
    prev = 0
    for e, end in enumerate(off.tolist()):
        h = inp[prev:end].float() @ w[e].float().t()
        if form == "swiglu":
            h = h[:, :N] * torch.nn.functional.silu(h[:, N:])
        ref[prev:end] = h
        prev = end
    if form != "swiglu":
        scattered = torch.empty_like(ref)
        scattered[ss.long()] = ref
        ref = scattered
    assert_close_scaled(split, ref, torch.bfloat16, rtol=2e-2, atol=2e-2, what=f"split-K {form} {name}")
    # against the unsplit kernel: the fp32 sums differ in their last bits only, which flips a bf16 rounding now and then
    differ = (split != whole)
    assert differ.float().mean().item() < 2e-3
    # (one bf16 step of the value, or -- for results next to zero -- the reordering error of the fp32 sum itself)
    one_step = (split.float() - whole.float()).abs() <= whole.float().abs() * 2 ** -7 + 1e-4
    assert bool(one_step.all())


def test_split_k_workspace_outlives_a_captured_graph(device):
    """A product long enough to be cut along K (K >= 5120) is captured into a HIP graph, which bakes the address of
    the workspace into the graph.  Calls on more than sixteen further streams must neither release that buffer nor
    hand it to someone else: every later replay still equals the eager result, also after the caching allocator
    has been churned.  Shorter contractions never get a workspace."""
    ops = _ops()
    counts, K, N = [5000, 5000, 5000, 5000], 8192, 1024
    g = torch.Generator().manual_seed(77)
    E, L = len(counts), sum(counts)
    off = torch.tensor(counts).cumsum(0).to(torch.int32).to(device)
    ss = torch.randperm(L, generator=g).to(torch.int32).to(device)
    inp = (torch.randn(L, K, generator=g) * 0.5).to(torch.bfloat16).to(device)
    w = (torch.randn(E, N, K, generator=g) * 0.05).to(torch.bfloat16).to(device)
    print("split-K workspace under graph capture", flush=True)
    assert ops._gemm_workspace(torch.device(device), 512, torch.bfloat16)[0] is None
    assert ops._gemm_workspace(torch.device(device), 8192, torch.float32)[0] is None
    eager = ops.scattered_gemm(inp, w, 1, ss, off, True, False, cfg=7)
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.scattered_gemm(inp, w, 1, ss, off, True, False, cfg=7)   # creates the side stream's workspace
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ops.scattered_gemm(inp, w, 1, ss, off, True, False, cfg=7)
    held = {k: v.data_ptr() for k, v in ops._GEMM_WS.items()}
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, eager)

    small_in = inp[:, :5120].contiguous()
    small_w = w[:, :256, :5120].contiguous()
    for i in range(20):   # more streams than the cache keeps buffers for
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            ops.scattered_gemm(small_in, small_w, 1, ss, off, True, False, cfg=7)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        junk = torch.full((96 << 20,), 0x7f, dtype=torch.uint8, device=device)  # would land on a released workspace
        del junk
        if i % 5 == 4:
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay after {i + 1} further streams"
    for k, ptr in held.items():   # nothing that existed at capture time was dropped or replaced
        assert ops._GEMM_WS[k].data_ptr() == ptr
    assert len(ops._GEMM_WS) <= ops._GEMM_WS_MAX


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_persistent_kernel_random_shapes(device, seed):
    """The persistent kernel's scheduling (tile order by XCD in both forms, last round cut along K, finishing
    launch, grids smaller than the chip) on random shapes: expert counts from 1 to 130 with empty experts, row
    counts around the tile edge and up to 66000, contraction lengths from 128 to 8192, 1 to 10 column tiles,
    all three forms -- against an fp32 product of the same rounded operands."""
    import random

    ops = _ops()
    rnd = random.Random(seed)
    # one shape that once lost tiles: 20 tiles on a grid of 40 (an odd number of slots per XCD), cut in two along K
    fixed = [(3, 256, 8192, 2400, "plain", [128, 0, 128])] if seed == 2 else []
    for case in range(24):
        fixed_counts = None
        if case < len(fixed):
            E, L, K, N, form, fixed_counts = fixed[case]
        else:
            E = rnd.choice([1, 2, 3, 8, 40, 64, 65, 130])
            K = 32 * rnd.choice([4, 5, 16, 33, 48, 128, 160, 192, 256])
            form = rnd.choice(["plain", "plain", "swiglu", "weight_kn"])
            N = 8 * rnd.choice([1, 16, 31, 32, 64, 96, 128, 256, 300])
            L = rnd.choice([1, 255, 256, 257, 3000, 10000, 30000, 66000])
        rows_w = 2 * N if form == "swiglu" else N
        if L * K * 2 > 1.2e9 or E * rows_w * K * 2 > 1.5e9:
            continue
        g = torch.Generator().manual_seed(seed * 100003 + case)
        p = torch.rand(E, generator=g).pow(rnd.choice([0.5, 3.0, 6.0]))
        if E > 2:
            p[torch.rand(E, generator=g) < 0.2] = 0
        if p.sum() == 0:
            p[0] = 1
        counts = torch.bincount(torch.multinomial(p.double(), L, replacement=True, generator=g), minlength=E)
        if fixed_counts is not None:
            counts = torch.tensor(fixed_counts)
        off = counts.cumsum(0).to(torch.int32).to(device)
        ss = torch.randperm(L, generator=g).to(torch.int32).to(device)
        inp = (torch.randn(L, K, generator=g) * 0.5).to(torch.bfloat16).to(device)
        w = (torch.randn(E, rows_w, K, generator=g) * (2.0 / K ** 0.5)).to(torch.bfloat16).to(device)
        print(f"persistent kernel seed {seed} case {case}: E={E} L={L} K={K} N={N} {form}", flush=True)
        if form == "swiglu":
            out = ops.up_swiglu(inp, w, 1, torch.arange(L, dtype=torch.int32, device=device), off, cfg=7)
        elif form == "weight_kn":
            out = ops.scattered_gemm(inp, w.transpose(1, 2).contiguous(), 1, ss, off, True, False, weight_kn=True)
        else:
            out = ops.scattered_gemm(inp, w, 1, ss, off, True, False, cfg=7)
        ref = torch.zeros((L, N), dtype=torch.float32, device=device)
        prev = 0
        for e, end in enumerate(off.tolist()):
            if end > prev:
                h = inp[prev:end].float() @ w[e].float().t()
                ref[prev:end] = h[:, :N] * torch.nn.functional.silu(h[:, N:]) if form == "swiglu" else h
            prev = end
        if form != "swiglu":
            scattered = torch.empty_like(ref)
            scattered[ss.long()] = ref
            ref = scattered
        err = (out.float() - ref).abs().max().item()
        assert err <= 1e-2 * ref.abs().max().item() + 1e-3, (case, E, L, K, N, form, err)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,k,H", [(1, 1, 8), (15, 8, 32), (512, 2, 256), (100, 6, 4096), (77, 3, 100), (300, 8, 1536)])
def test_combine(device, dtype, T, k, H):
    ops = _ops()
    g = torch.Generator().manual_seed(T + k + H)
    o = _rand((T * k, H), 1.0, dtype, g)
    gates = torch.softmax(torch.randn(T, k, generator=g), -1).to(dtype)
    y = ops.combine(o.to(device), gates.to(device))
    ref = torch.einsum("tk,tkh->th", gates.float(), o.float().view(T, k, H))
    tol = {torch.float32: dict(rtol=1e-5, atol=1e-6), torch.bfloat16: dict(rtol=8e-3, atol=1e-3),
           torch.float16: dict(rtol=1e-3, atol=1e-4)}[dtype]
    torch.testing.assert_close(y.cpu().float(), ref, **tol)


def test_scattered_experts_signature_with_gates(device):
    """The drop-in entry: (E, in, out) permuted view, int64 indices, gates contraction."""
    ops = _ops()
    g = torch.Generator().manual_seed(11)
    T, E, k, H, I = 128, 8, 2, 64, 96
    se, ss, off = _routing(T, E, k, seed=2)
    a = _rand((T * k, I), 1.0, torch.bfloat16, g)
    w = _rand((E, H, I), 0.1, torch.bfloat16, g)
    gates = torch.softmax(torch.randn(T, k, generator=g), -1).to(torch.bfloat16)
    y = ops.scattered_experts(inputs=a.to(device), expert_weights=w.to(device).permute(0, 2, 1), k=1,
                              sorted_expert_idxs=se.to(device), sorted_scattered_idxs=ss.to(device),
                              expert_offsets=off.to(device), gates=gates.to(device), grouped_in=True)
    ref = oracle.scattered_experts_oracle(a, w, 1, se, ss, off, gates=gates, grouped_in=True)
    torch.testing.assert_close(y.cpu().float(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,H,I", [(64, 64, 6, 4096, 1408), (8, 8, 2, 256, 128), (1, 4, 1, 64, 32),
                                       (200, 4, 2, 1024, 208), (40, 16, 4, 2048, 64)])
def test_fp8_up_down(device, dtype, T, E, k, H, I):
    if dtype == torch.float16 and H * I > 2**21:
        pytest.skip("the full decode shape is run once, in bf16")
    ops = _ops()
    g = torch.Generator().manual_seed(T + H)
    se, ss, off = _routing(T, E, k, seed=T + 1)
    x = _rand((T, H), 1.0, dtype, g)
    w_fc_q, fc_scale = oracle.quantize_fp8_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w_pj_q, pj_scale = oracle.quantize_fp8_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    print(f"fp8 T={T} E={E} k={k} H={H} I={I} {dtype}", flush=True)
    act = ops.up_swiglu_fp8(x.to(device), w_fc_q.to(device), fc_scale.to(device), k, ss.to(device), off.to(device), widen=False, cfg=0)
    w_fc = oracle.dequant_fp8(w_fc_q, fc_scale)
    ref_act = oracle.swiglu(oracle.scattered_experts_oracle(x, w_fc, k, se, ss, off, grouped_out=True))
    torch.testing.assert_close(act.cpu().float(), ref_act, rtol=2e-2, atol=2e-3)
    o = ops.down_fp8(act, w_pj_q.to(device), pj_scale.to(device), ss.to(device), off.to(device), widen=False, cfg=0)
    w_pj = oracle.dequant_fp8(w_pj_q, pj_scale)
    ref_o = oracle.scattered_experts_oracle(act.cpu(), w_pj, 1, se, ss, off, grouped_in=True)
    torch.testing.assert_close(o.cpu().float(), ref_o, rtol=2e-2, atol=2e-3)


@pytest.mark.parametrize("T,E,k,H,I", [(64, 64, 6, 4096, 1408), (40, 8, 2, 512, 264), (300, 4, 2, 256, 128)])
def test_fp8_tiled_layout_is_bit_identical(device, T, E, k, H, I):
    """The streamed-tile weight layout changes the HBM access pattern only: same bits out as row-major weights
    (incl. a channel count that is not a multiple of the unit size, and experts with more than 16 rows).
    With K < 512 the row-major weights run the older kernel, so there the two agree to rounding only."""
    ops = _ops()
    g = torch.Generator().manual_seed(T + I)
    se, ss, off = _routing(T, E, k, seed=3)
    x = _rand((T, H), 1.0, torch.bfloat16, g).to(device)
    w_fc_q, fc_scale = oracle.quantize_fp8_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w_pj_q, pj_scale = oracle.quantize_fp8_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    w_fc_q, fc_scale, w_pj_q, pj_scale = (t.to(device) for t in (w_fc_q, fc_scale, w_pj_q, pj_scale))
    ss, off = ss.to(device), off.to(device)
    fc_t = ops.fp8_tile(w_fc_q, glu=True)
    assert torch.equal(ops.fp8_untile(fc_t, E, 2 * I, H, True).view(torch.uint8), w_fc_q.view(torch.uint8))
    act = ops.up_swiglu_fp8(x, w_fc_q, fc_scale, k, ss, off, widen=False, cfg=0)
    act_t = ops.up_swiglu_fp8(x, fc_t, fc_scale, k, ss, off, widen=False, cfg=0)
    if H >= 512:
        assert torch.equal(act, act_t)
    else:  # row-major weights with a short K take the older kernel, which sums in another order
        torch.testing.assert_close(act_t.float(), act.float(), rtol=2e-2, atol=1e-3)
        act = act_t
    if I % 128 == 0:
        pj_t = ops.fp8_tile(w_pj_q, glu=False)
        assert torch.equal(ops.fp8_untile(pj_t, E, H, I, False).view(torch.uint8), w_pj_q.view(torch.uint8))
        o = ops.down_fp8(act, w_pj_q, pj_scale, ss, off, widen=False, cfg=0)
        o_t = ops.down_fp8(act, pj_t, pj_scale, ss, off, widen=False, cfg=0)
        if I >= 512:
            assert torch.equal(o, o_t)
        else:
            torch.testing.assert_close(o_t.float(), o.float(), rtol=2e-2, atol=1e-3)
    else:
        with pytest.raises(ValueError):
            ops.fp8_tile(w_pj_q, glu=False)


@pytest.mark.parametrize("T,E,k,H,I,skew", [(100, 64, 2, 1024, 512, True), (8, 4, 1, 512, 384, False),
                                            (37, 16, 3, 2048, 640, True), (9, 40, 1, 384, 1024, False),
                                            (250, 130, 4, 512, 384, True)])
def test_fp8_few_rows_per_expert(device, T, E, k, H, I, skew):
    """The decode regime (at most 8 rows per expert on average) with skewed routing: experts with many times 8
    rows (several passes of the streaming kernel over one unit) next to experts without any; the smallest case
    has exactly 8 slots.  Tiled weights must give the bits of the row-major weights where both run the same
    arithmetic (K >= 512), and both must match the oracle."""
    ops = _ops()
    g = torch.Generator().manual_seed(T * 7 + E)
    se, ss, off = _routing(T, E, k, seed=T + E, skew=skew)
    counts = torch.diff(off, prepend=torch.zeros(1, dtype=off.dtype))
    assert T * k <= 8 * E and T * k >= 8
    if skew:
        assert counts.max().item() > 16 and counts.min().item() == 0
    x = _rand((T, H), 1.0, torch.bfloat16, g)
    w_fc_q, fc_scale = oracle.quantize_fp8_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w_pj_q, pj_scale = oracle.quantize_fp8_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    print(f"fp8 few rows T={T} E={E} k={k} H={H} I={I} max rows {counts.max().item()}", flush=True)
    xd, ssd, offd = x.to(device), ss.to(device), off.to(device)
    fc_d, fcs_d, pj_d, pjs_d = (t.to(device) for t in (w_fc_q, fc_scale, w_pj_q, pj_scale))
    act_t = ops.up_swiglu_fp8(xd, ops.fp8_tile(fc_d, glu=True), fcs_d, k, ssd, offd, widen=False, cfg=0)
    act_r = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False, cfg=0)
    if H >= 512:
        assert torch.equal(act_t, act_r)
    ref_act = oracle.swiglu(oracle.scattered_experts_oracle(x, oracle.dequant_fp8(w_fc_q, fc_scale), k, se, ss, off,
                                                            grouped_out=True))
    torch.testing.assert_close(act_t.cpu().float(), ref_act, rtol=2e-2, atol=2e-3)
    o_t = ops.down_fp8(act_t, ops.fp8_tile(pj_d, glu=False), pjs_d, ssd, offd, widen=False, cfg=0)
    o_r = ops.down_fp8(act_t, pj_d, pjs_d, ssd, offd, widen=False, cfg=0)
    if I >= 512:
        assert torch.equal(o_t, o_r)
    ref_o = oracle.scattered_experts_oracle(act_t.cpu(), oracle.dequant_fp8(w_pj_q, pj_scale), 1, se, ss, off,
                                            grouped_in=True)
    torch.testing.assert_close(o_t.cpu().float(), ref_o, rtol=2e-2, atol=2e-3)
    torch.testing.assert_close(o_r.cpu().float(), ref_o, rtol=2e-2, atol=2e-3)


def test_fp8_all_bit_patterns(device):
    """Every e4m3fn byte value is widened exactly: K=256 one-hot activations read out each pattern."""
    ops = _ops()
    E, k, T = 1, 1, 16
    H = 256
    I = 16
    codes = torch.arange(256, dtype=torch.uint8)
    finite = ~torch.isnan(codes.view(torch.float8_e4m3fn).float())
    wq = torch.zeros(E, H, 256, dtype=torch.uint8)  # down weights (E, out=H, in=I') with I' = 256
    wq[0, :, :] = codes  # every output channel holds all 256 codes along K
    wq[0, :, ~finite] = 0
    scale = torch.ones(E, H)
    se, ss, off = oracle.sort_bin(torch.zeros(T, 1, dtype=torch.long), E)
    eye_rows = torch.zeros(T, 256, dtype=torch.bfloat16)
    for base in range(0, 256, T):
        eye_rows.zero_()
        for r in range(T):
            eye_rows[r, base + r] = 1.0
        o = ops.down_fp8(eye_rows.to(device), wq.view(torch.float8_e4m3fn).to(device), scale.to(device),
                         ss.to(device), off.to(device))
        got = o.cpu().float()[:, 0]
        want = codes[base:base + T].view(torch.float8_e4m3fn).float()
        want = torch.where(finite[base:base + T], want, torch.zeros_like(want))
        assert torch.equal(got, want.to(torch.bfloat16).float()), f"codes {base}..{base + T}"


@pytest.mark.parametrize("seed", [1, 2])
def test_fp8_random_shapes(device, seed):
    """The fp8 kernels on random shapes and routings: 1 to 257 tokens, 1 to 64 experts (some without rows, some with
    many times 8), hidden and intermediate sizes from 128 to 2048 in steps of 128 (one to sixteen ring stages, so
    both the short-ring path and the counted tail), both 16-bit types.  Tiled and row-major weights must agree bit
    for bit where both run the streaming kernel (K >= 512), and both must match the oracle; the tile kernels run
    the same problems (bit-identical from either weight layout, same bounds against the oracle)."""
    import random

    ops = _ops()
    rnd = random.Random(seed)
    for case in range(20):
        E = rnd.choice([1, 2, 4, 8, 16, 33, 64])
        k = min(rnd.choice([1, 2, 4, 6, 8]), E)
        T = rnd.choice([1, 2, 5, 8, 16, 33, 64, 100, 257])
        H = 128 * rnd.choice([1, 2, 3, 4, 8, 11, 16])
        I = 128 * rnd.choice([1, 2, 3, 4, 5, 11])
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        g = torch.Generator().manual_seed(seed * 100003 + case * 7919 + E)
        noise = torch.rand(T, E, generator=g) + torch.arange(E).float().pow(1.3) * rnd.choice([0.0, 0.03, 0.2])
        se, ss, off = oracle.sort_bin(noise.argsort(dim=1)[:, :k], E)
        x = _rand((T, H), 1.0, dtype, g)
        w_fc_q, fc_scale = oracle.quantize_fp8_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
        w_pj_q, pj_scale = oracle.quantize_fp8_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
        xd, ssd, offd = x.to(device), ss.to(device), off.to(device)
        fc_d, fcs_d, pj_d, pjs_d = (t.to(device) for t in (w_fc_q, fc_scale, w_pj_q, pj_scale))
        print(f"fp8 random seed {seed} case {case}: T={T} E={E} k={k} H={H} I={I} {dtype}", flush=True)
        act_t = ops.up_swiglu_fp8(xd, ops.fp8_tile(fc_d, glu=True), fcs_d, k, ssd, offd, widen=False, cfg=0)
        act_r = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False, cfg=0)
        o_t = ops.down_fp8(act_t, ops.fp8_tile(pj_d, glu=False), pjs_d, ssd, offd, widen=False, cfg=0)
        o_r = ops.down_fp8(act_t, pj_d, pjs_d, ssd, offd, widen=False, cfg=0)
        if H >= 512:
            assert torch.equal(act_t, act_r), (case, "up")
        if I >= 512:
            assert torch.equal(o_t, o_r), (case, "down")
        ref_act = oracle.swiglu(oracle.scattered_experts_oracle(x, oracle.dequant_fp8(w_fc_q, fc_scale), k, se, ss, off,
                                                                grouped_out=True))
        ref_o = oracle.scattered_experts_oracle(act_t.cpu(), oracle.dequant_fp8(w_pj_q, pj_scale), 1, se, ss, off,
                                                grouped_in=True)
        # the tile kernels on the same problem (tiled and row-major weights: the same bits)
        act_k = ops.up_swiglu_fp8(xd, ops.fp8_tile(fc_d, glu=True), fcs_d, k, ssd, offd, widen=False, cfg=1)
        assert torch.equal(act_k, ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False, cfg=1)), (case, "up tiles")
        o_k = ops.down_fp8(act_t, ops.fp8_tile(pj_d, glu=False), pjs_d, ssd, offd, widen=False, cfg=1)
        assert torch.equal(o_k, ops.down_fp8(act_t, pj_d, pjs_d, ssd, offd, widen=False, cfg=1)), (case, "down tiles")
        for name, got, ref in (("up", act_t, ref_act), ("up row-major", act_r, ref_act), ("down", o_t, ref_o),
                               ("down row-major", o_r, ref_o), ("up tile kernels", act_k, ref_act),
                               ("down tile kernels", o_k, ref_o)):
            err = (got.cpu().float() - ref).abs().max().item()
            assert err <= 2e-2 * ref.abs().max().item() + 2e-3, (case, name, err)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("E,R,K,glu", [(3, 64, 256, True), (2, 40, 128, True), (5, 96, 384, False),
                                       (2, 50, 256, False), (1, 8, 48, False), (2, 12, 80, True)])
def test_fp8_dequant(device, dtype, E, R, K, glu):
    """The widened weights are round(w * scale) bit for bit, from the row-major and from the tiled layout (channel
    counts that do not fill the last unit of 16 / 32 included)."""
    ops = _ops()
    g = torch.Generator().manual_seed(E * 1000 + R + K)
    w_q, scale = oracle.quantize_fp8_per_channel(torch.randn(E, R, K, generator=g) * 0.02)
    want = (w_q.float() * scale[:, :, None]).to(dtype)
    print(f"fp8 dequant E={E} R={R} K={K} glu={glu} {dtype}", flush=True)
    got = ops.fp8_dequant(w_q.to(device), scale.to(device), K, glu, dtype)
    assert got.dtype == dtype and tuple(got.shape) == (E, R, K)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    if K % 128 == 0:
        tiled = ops.fp8_tile(w_q.to(device), glu)
        got_t = ops.fp8_dequant(tiled, scale.to(device), K, glu, dtype)
        assert torch.equal(got_t.cpu().view(torch.int16), want.view(torch.int16))


def test_fp8_dequant_all_bit_patterns(device):
    """Every finite e4m3fn byte value, widened with a scale of one and with one that is not a power of two."""
    ops = _ops()
    codes = torch.arange(256, dtype=torch.uint8)
    finite = ~torch.isnan(codes.view(torch.float8_e4m3fn).float())
    row = torch.where(finite, codes, torch.zeros_like(codes))
    w_q = row.repeat(2, 16, 1).contiguous().view(torch.float8_e4m3fn)       # (2, 16, 256)
    for sc in (1.0, 0.37):
        scale = torch.full((2, 16), sc)
        for dtype in (torch.bfloat16, torch.float16):
            want = (w_q.float() * scale[:, :, None]).to(dtype)
            for src in (w_q.to(device), ops.fp8_tile(w_q.to(device), False)):
                got = ops.fp8_dequant(src, scale.to(device), 256, False, dtype)
                bad = (got.cpu().view(torch.int16) != want.view(torch.int16)).nonzero()
                assert bad.numel() == 0, (sc, dtype, src.dim(), bad[:8].tolist(),
                                          [(float(got[tuple(b)]), float(want[tuple(b)])) for b in bad[:8]])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,H,I", [(300, 4, 2, 256, 128), (1024, 8, 2, 512, 272), (513, 3, 1, 384, 96),
                                       (1600, 2, 1, 256, 128)])
def test_fp8_widened_weights_for_many_rows(device, dtype, T, E, k, H, I):
    """With very many rows per expert the fp8 calls widen the weights and run the persistent 16-bit kernels: same
    contract against the oracle, agreement with the fp8 kernels to rounding, and the automatic choice from 768 rows
    per expert on.
    The widened weights are rounded to the activation dtype (2^-9 relative in bf16, beside the 2^-4 of e4m3 itself),
    which the fp8 kernels' weights are not: the absolute bound is twice that of the fp8 kernels' tests."""
    ops = _ops()
    atol = 4e-3 if dtype == torch.bfloat16 else 2e-3
    g = torch.Generator().manual_seed(T + H + I)
    se, ss, off = _routing(T, E, k, seed=T + 3)
    x = _rand((T, H), 1.0, dtype, g)
    w_fc_q, fc_scale = oracle.quantize_fp8_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w_pj_q, pj_scale = oracle.quantize_fp8_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    xd, ssd, offd = x.to(device), ss.to(device), off.to(device)
    fc_d, fcs_d, pj_d, pjs_d = w_fc_q.to(device), fc_scale.to(device), w_pj_q.to(device), pj_scale.to(device)
    auto_widens = T * k >= ops.FP8_DENSE_ROWS_PER_EXPERT * E
    print(f"fp8 widened T={T} E={E} k={k} H={H} I={I} {dtype} auto={auto_widens}", flush=True)
    act = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=True)
    auto = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd)
    assert torch.equal(auto, act if auto_widens else ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False))
    ref_act = oracle.swiglu(oracle.scattered_experts_oracle(x, oracle.dequant_fp8(w_fc_q, fc_scale), k, se, ss, off,
                                                           grouped_out=True))
    torch.testing.assert_close(act.cpu().float(), ref_act, rtol=2e-2, atol=atol)
    act_fp8 = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False, cfg=0)
    torch.testing.assert_close(act.float(), act_fp8.float(), rtol=2e-2, atol=atol)
    o = ops.down_fp8(act, pj_d, pjs_d, ssd, offd, widen=True)
    auto = ops.down_fp8(act, pj_d, pjs_d, ssd, offd)
    assert torch.equal(auto, o if auto_widens else ops.down_fp8(act, pj_d, pjs_d, ssd, offd, widen=False))
    ref_o = oracle.scattered_experts_oracle(act.cpu(), oracle.dequant_fp8(w_pj_q, pj_scale), 1, se, ss, off,
                                            grouped_in=True)
    torch.testing.assert_close(o.cpu().float(), ref_o, rtol=2e-2, atol=atol)
    o_fp8 = ops.down_fp8(act, pj_d, pjs_d, ssd, offd, widen=False, cfg=0)
    torch.testing.assert_close(o.float(), o_fp8.float(), rtol=2e-2, atol=atol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,H,I", [(8, 4, 1, 256, 128), (100, 4, 2, 1024, 208), (300, 4, 2, 256, 128),
                                       (1024, 8, 2, 512, 272), (2100, 2, 1, 384, 112), (37, 16, 3, 2048, 640),
                                       (600, 5, 1, 128, 80)])
def test_fp8_tile_kernels(device, dtype, T, E, k, H, I):
    """fp8 weights on the grouped GEMM's tile kernels (bytes widened on their way into LDS, scale in the epilogue):
    the oracle's contract, bit-identical from the row-major and the tiled layout, equal to the streaming kernels up
    to rounding; all three tile shapes (by rows per expert), partial K tiles, experts without rows.  The automatic
    choice is the tile kernels from 16 rows per expert on average, the streaming kernels below."""
    ops = _ops()
    g = torch.Generator().manual_seed(T * 3 + H + I)
    se, ss, off = _routing(T, E, k, seed=T + 5)
    x = _rand((T, H), 1.0, dtype, g)
    w_fc_q, fc_scale = oracle.quantize_fp8_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w_pj_q, pj_scale = oracle.quantize_fp8_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    xd, ssd, offd = x.to(device), ss.to(device), off.to(device)
    fc_d, fcs_d, pj_d, pjs_d = w_fc_q.to(device), fc_scale.to(device), w_pj_q.to(device), pj_scale.to(device)
    print(f"fp8 tiles T={T} E={E} k={k} H={H} I={I} {dtype}", flush=True)
    act = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False, cfg=1)
    ref_act = oracle.swiglu(oracle.scattered_experts_oracle(x, oracle.dequant_fp8(w_fc_q, fc_scale), k, se, ss, off,
                                                           grouped_out=True))
    torch.testing.assert_close(act.cpu().float(), ref_act, rtol=2e-2, atol=2e-3)
    act_s = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False, cfg=0)
    torch.testing.assert_close(act.float(), act_s.float(), rtol=2e-2, atol=2e-3)
    if H % 128 == 0:
        assert torch.equal(ops.up_swiglu_fp8(xd, ops.fp8_tile(fc_d, glu=True), fcs_d, k, ssd, offd, widen=False, cfg=1), act)
    auto = ops.up_swiglu_fp8(xd, fc_d, fcs_d, k, ssd, offd, widen=False)
    assert torch.equal(auto, act if T * k >= 16 * E else act_s)

    o = ops.down_fp8(act, pj_d, pjs_d, ssd, offd, widen=False, cfg=1)
    ref_o = oracle.scattered_experts_oracle(act.cpu(), oracle.dequant_fp8(w_pj_q, pj_scale), 1, se, ss, off,
                                            grouped_in=True)
    torch.testing.assert_close(o.cpu().float(), ref_o, rtol=2e-2, atol=2e-3)
    o_s = ops.down_fp8(act, pj_d, pjs_d, ssd, offd, widen=False, cfg=0)
    torch.testing.assert_close(o.float(), o_s.float(), rtol=2e-2, atol=2e-3)
    if I % 128 == 0:
        assert torch.equal(ops.down_fp8(act, ops.fp8_tile(pj_d, glu=False), pjs_d, ssd, offd, widen=False, cfg=1), o)
    auto = ops.down_fp8(act, pj_d, pjs_d, ssd, offd, widen=False)
    assert torch.equal(auto, o if T * k >= 16 * E else o_s)


def test_inner_loop_probes_run(device):
    """The diagnostic kernels behind bench.py's `ceilings.gemm_inner_loop` (mi_moe_probe_kloop): every mode runs to
    completion on a short loop, writes its whole sink, and the matrix modes agree with each other -- modes 0, 1 and 3
    multiply the same first ring contents when the data repeats every 64 bytes of K."""
    from dolomite_engine_amd import _lib

    lib = _lib.load()
    n = (2 << 20) // 2 + 4096
    data = torch.full((n,), 0.5, dtype=torch.bfloat16, device=device)   # constant data: every slice is the same
    sink_bytes = lib.mi_moe_probe_sink_bytes()
    assert sink_bytes > 0 and sink_bytes % (512 * 4) == 0
    stream = torch.cuda.current_stream().cuda_stream
    sums = {}
    for mode in (0, 1, 2, 3):
        sink = torch.full((sink_bytes // 4,), float("nan"), dtype=torch.float32, device=device)
        print(f"probe mode {mode}", flush=True)
        rc = lib.mi_moe_probe_kloop(mode, data.data_ptr(), n * 2, 64, sink.data_ptr(), sink_bytes, stream)
        assert rc == 0, lib.mi_moe_strerror(rc).decode()
        torch.cuda.synchronize()
        assert bool(torch.isfinite(sink).all())
        sums[mode] = sink.clone()
    # 64 slices x 32 k of 0.5 * 0.5 per output element, 128 elements summed per thread
    want = 64 * 32 * 0.25 * 128
    for mode in (0, 1, 3):
        assert bool((sums[mode] == want).all()), mode
