"""Pins the CPU oracle (oracle/moe_oracle.py) WITHOUT using its own formulas.

Each oracle function is checked against something the oracle did not produce: golden vectors from an
independent implementation (transformers' GraniteMoe, see tests/golden/make_golden.py), brute force in
pure Python / float64 numpy, closed forms, special cases that reduce to a library routine, and
invariants.  The checks are chosen so that a dropped term, a swapped GLU half, a wrong index or a
transposed operand fails at least one of them.
"""

import glob
import itertools
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as oracle

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "granitemoe_*.npz")))


# ---------------------------------------------------------------------------------------------------
# golden vectors from the independent implementation
# ---------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_layer_matches_independent_implementation(path):
    z = np.load(path)
    x, gate_w, w_fc, w_proj = (torch.from_numpy(z[n]) for n in ("x", "gate_w", "w_fc", "w_proj"))
    k = int(z["k"])
    out = oracle.moe_forward(x, gate_w, w_fc, w_proj, k)
    assert torch.equal(out.experts, torch.from_numpy(z["topk_idx"]))
    torch.testing.assert_close(out.logits, torch.from_numpy(z["logits"]), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.gates, torch.from_numpy(z["gates"]), rtol=1e-6, atol=1e-7)
    # the reference's own bar for "eager == transformers" is atol 3e-7 on logits of size ~1
    torch.testing.assert_close(out.y, torch.from_numpy(z["y"]), rtol=1e-5, atol=3e-7)


def test_golden_files_present():
    assert len(GOLDEN) == 2


def test_glu_half_order_matters_on_golden():
    """Swapping [up ; gate] must break the golden comparison (guards against a symmetric bug)."""
    z = np.load(GOLDEN[0])
    x, gate_w, w_fc, w_proj = (torch.from_numpy(z[n]) for n in ("x", "gate_w", "w_fc", "w_proj"))
    up, gate = w_fc.chunk(2, dim=1)
    swapped = torch.cat([gate, up], dim=1)
    out = oracle.moe_forward(x, gate_w, swapped, w_proj, int(z["k"]))
    assert (out.y - torch.from_numpy(z["y"])).abs().max() > 1e-3


# ---------------------------------------------------------------------------------------------------
# router
# ---------------------------------------------------------------------------------------------------


def test_router_logits_closed_form_float64():
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = torch.randn(37, 48, generator=g).to(dtype)
        w = (torch.randn(9, 48, generator=g) * 0.1).to(dtype)
        b = torch.randn(9, generator=g)
        exact = x.double().numpy() @ w.double().numpy().T
        got = oracle.router_logits(x, w)
        assert got.dtype == dtype
        want = torch.from_numpy(exact).to(dtype)  # one rounding of the exact product
        ulp = {torch.float32: 1e-6, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
        torch.testing.assert_close(got.float(), want.float(), rtol=ulp, atol=ulp)
        got_b = oracle.router_logits(x, w, b)
        want_b = (got.double() + b.double()).to(dtype)
        torch.testing.assert_close(got_b.float(), want_b.float(), rtol=ulp, atol=ulp)


def _brute_topk(row, k):
    """Pure-python selection: repeatedly take the largest value, lowest index on ties."""
    taken, out = set(), []
    for _ in range(k):
        best = None
        for i, v in enumerate(row):
            if i in taken:
                continue
            if best is None or v > row[best]:
                best = i
        taken.add(best)
        out.append(best)
    return out


@pytest.mark.parametrize("E,k", [(8, 2), (8, 8), (5, 1), (40, 8), (64, 6)])
def test_topk_brute_force_with_ties(E, k):
    g = torch.Generator().manual_seed(E * 10 + k)
    logits = torch.round(torch.randn(200, E, generator=g) * 2) / 2  # many exact ties
    vals, idx = oracle.topk_canonical(logits, k)
    for r in range(logits.shape[0]):
        want = _brute_topk(logits[r].tolist(), k)
        assert idx[r].tolist() == want
        assert vals[r].tolist() == [logits[r, i].item() for i in want]


def test_topk_agrees_with_torch_on_tie_free_rows():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(500, 40, generator=g)  # fp32 gaussian: ties have probability ~0
    vals, idx = oracle.topk_canonical(logits, 8)
    tv, ti = logits.topk(8, dim=-1)
    assert torch.equal(idx, ti) and torch.equal(vals, tv)
    # k == 1 is max(): first occurrence
    one = torch.tensor([[1.0, 3.0, 3.0, 2.0]])
    assert oracle.topk_canonical(one, 1)[1].tolist() == [[1]]
    assert one.max(dim=-1, keepdim=True)[1].tolist() == [[1]]


def test_softmax_topk_closed_form_and_invariants():
    g = torch.Generator().manual_seed(4)
    vals = torch.sort(torch.randn(64, 8, generator=g), dim=-1, descending=True).values
    got = oracle.softmax_topk(vals, torch.float32)
    v64 = vals.double().numpy()
    e = np.exp(v64 - v64.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(got.numpy(), want, rtol=2e-6, atol=1e-7)
    assert np.allclose(got.sum(-1).numpy(), 1.0, atol=1e-6)
    assert (got[:, :-1] >= got[:, 1:]).all()  # gates follow the order of the logits
    # equal logits -> uniform gates 1/k
    assert torch.allclose(oracle.softmax_topk(torch.zeros(3, 4), torch.float32), torch.full((3, 4), 0.25))
    assert oracle.softmax_topk(vals.bfloat16(), torch.bfloat16).dtype == torch.bfloat16


# ---------------------------------------------------------------------------------------------------
# sort / bin
# ---------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("T,k,E", [(1, 1, 1), (15, 8, 8), (100, 2, 8), (1024, 4, 40), (7, 3, 64)])
def test_sort_bin_against_numpy_stable_argsort(T, k, E):
    g = torch.Generator().manual_seed(T + k + E)
    sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    se, ss, off = oracle.sort_bin(sel, E)
    flat = sel.flatten().numpy()
    order = np.argsort(flat, kind="stable")
    assert np.array_equal(ss.numpy(), order)
    assert np.array_equal(se.numpy(), flat[order])
    assert np.array_equal(off.numpy(), np.cumsum(np.bincount(flat, minlength=E)))
    # invariants
    assert (np.diff(se.numpy()) >= 0).all()
    assert sorted(ss.tolist()) == list(range(T * k))
    assert off[-1].item() == T * k
    for e in range(E):  # within an expert the slots are ascending (stable)
        lo = 0 if e == 0 else off[e - 1].item()
        assert (np.diff(ss[lo:off[e].item()].numpy()) > 0).all()


def test_expert_assignment_matches_sort_bin():
    g = torch.Generator().manual_seed(9)
    sel = torch.rand(50, 8, generator=g).argsort(dim=1)[:, :3]
    gates = torch.rand(50, 3, generator=g)
    bi, bg, cnt = oracle.expert_assignment(gates, sel, 8)
    se, ss, off = oracle.sort_bin(sel, 8)
    assert torch.equal(bi, ss // 3)
    assert torch.equal(bg, gates.flatten()[ss])
    assert torch.equal(cnt.cumsum(0), off)


# ---------------------------------------------------------------------------------------------------
# experts
# ---------------------------------------------------------------------------------------------------


def _brute_layer(x, gates, sel, w_fc, w_proj):
    """Token-by-token float64 evaluation straight from the definition of the layer."""
    T, H = x.shape
    I = w_proj.shape[2]
    y = np.zeros((T, H))
    x, gates, w_fc, w_proj = (t.double().numpy() for t in (x, gates, w_fc, w_proj))
    for t in range(T):
        for j, e in enumerate(sel[t].tolist()):
            h = w_fc[e] @ x[t]
            up, gate = h[:I], h[I:]
            a = up * (gate / (1.0 + np.exp(-gate)))
            y[t] += gates[t, j] * (w_proj[e] @ a)
    return y


def test_experts_eager_float64_brute_force():
    g = torch.Generator().manual_seed(11)
    T, H, E, k, I = 23, 16, 6, 3, 10
    x = torch.randn(T, H, generator=g)
    w_fc = torch.randn(E, 2 * I, H, generator=g) * 0.3
    w_proj = torch.randn(E, H, I, generator=g) * 0.3
    sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    gates = torch.softmax(torch.randn(T, k, generator=g), -1)
    got = oracle.experts_eager(x, gates, sel, w_fc, w_proj)
    np.testing.assert_allclose(got.numpy(), _brute_layer(x, gates, sel, w_fc, w_proj), rtol=2e-5, atol=2e-6)


def test_single_expert_reduces_to_dense_swiglu_mlp():
    g = torch.Generator().manual_seed(12)
    T, H, I = 40, 24, 32
    x = torch.randn(T, H, generator=g)
    w_fc = torch.randn(1, 2 * I, H, generator=g) * 0.2
    w_proj = torch.randn(1, H, I, generator=g) * 0.2
    out = oracle.moe_forward(x, torch.zeros(1, H), w_fc, w_proj, 1)
    h = F.linear(x, w_fc[0])
    dense = F.linear(h[:, :I] * F.silu(h[:, I:]), w_proj[0])
    torch.testing.assert_close(out.y, dense, rtol=1e-5, atol=1e-6)
    assert torch.equal(out.gates, torch.ones(T, 1))


def test_identity_weights_give_permuted_rows():
    """scattered_experts with identity weights is a pure gather (and its inverse a pure scatter)."""
    g = torch.Generator().manual_seed(13)
    T, E, k, K = 30, 4, 2, 8
    x = torch.randn(T, K, generator=g)
    sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    se, ss, off = oracle.sort_bin(sel, E)
    eye = torch.eye(K).expand(E, K, K).contiguous()
    grouped = oracle.scattered_experts_oracle(x, eye, k, se, ss, off, grouped_out=True)
    assert torch.equal(grouped, x[ss // k])
    back = oracle.scattered_experts_oracle(grouped, eye, 1, se, ss, off, grouped_in=True)
    assert torch.equal(back, x.repeat_interleave(k, dim=0))


def test_scatter_pipeline_equals_eager_pipeline():
    """c_fc (grouped_out) -> SwiGLU -> c_proj (grouped_in, gates) is the eager gather/index_add layer."""
    g = torch.Generator().manual_seed(14)
    T, H, E, k, I = 64, 32, 8, 2, 48
    x = torch.randn(T, H, generator=g)
    w_fc = torch.randn(E, 2 * I, H, generator=g) * 0.2
    w_proj = torch.randn(E, H, I, generator=g) * 0.2
    sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    gates = torch.softmax(torch.randn(T, k, generator=g), -1)
    se, ss, off = oracle.sort_bin(sel, E)
    h = oracle.scattered_experts_oracle(x, w_fc, k, se, ss, off, grouped_out=True)
    y = oracle.scattered_experts_oracle(oracle.swiglu(h), w_proj, 1, se, ss, off, gates=gates, grouped_in=True)
    torch.testing.assert_close(y, oracle.experts_eager(x, gates, sel, w_fc, w_proj), rtol=1e-5, atol=1e-6)


def test_layer_is_linear_in_down_projection_and_gates():
    g = torch.Generator().manual_seed(15)
    T, H, E, k, I = 20, 16, 4, 2, 8
    x = torch.randn(T, H, generator=g)
    w_fc = torch.randn(E, 2 * I, H, generator=g) * 0.2
    w_proj = torch.randn(E, H, I, generator=g) * 0.2
    sel = torch.rand(T, E, generator=g).argsort(dim=1)[:, :k]
    gates = torch.softmax(torch.randn(T, k, generator=g), -1)
    y = oracle.experts_eager(x, gates, sel, w_fc, w_proj)
    assert torch.equal(oracle.experts_eager(x, gates, sel, w_fc, 2 * w_proj), 2 * y)
    assert torch.equal(oracle.experts_eager(x, 2 * gates, sel, w_fc, w_proj), 2 * y)


def test_reference_dtype_mode_keeps_dtype():
    g = torch.Generator().manual_seed(16)
    x = torch.randn(16, 32, generator=g).bfloat16()
    w_fc = (torch.randn(4, 64, 32, generator=g) * 0.1).bfloat16()
    w_proj = (torch.randn(4, 32, 32, generator=g) * 0.1).bfloat16()
    out32 = oracle.moe_forward(x, torch.randn(4, 32, generator=g).bfloat16(), w_fc, w_proj, 2)
    outbf = oracle.moe_forward(x, out32.logits.new_zeros(4, 32), w_fc, w_proj, 2, logits=out32.logits,
                               compute_dtype=None)
    assert out32.y.dtype == torch.float32 and outbf.y.dtype == torch.bfloat16
    torch.testing.assert_close(outbf.y.float(), out32.y, rtol=3e-2, atol=3e-3)


# ---------------------------------------------------------------------------------------------------
# aux loss, fp8
# ---------------------------------------------------------------------------------------------------


def test_switch_aux_loss_from_definition():
    g = torch.Generator().manual_seed(17)
    T, E, k = 12, 5, 2
    logits = torch.randn(T, E, generator=g)
    sel = logits.topk(k, dim=-1).indices
    lg = logits.double().numpy()
    p = np.exp(lg - lg.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    acc = p.sum(0)
    freq = np.bincount(sel.flatten().numpy(), minlength=E).astype(np.float64)
    switch = E * float(((acc / np.abs(acc).sum()) * (freq / np.abs(freq).sum())).sum())
    lse = np.log(np.exp(lg).sum(1))
    want = switch + 0.1 * float((lse ** 2).mean())
    assert math.isclose(oracle.switch_aux_loss(logits, sel).item(), want, rel_tol=1e-5)
    # perfectly balanced, uniform router: switch term is exactly 1
    uniform = torch.zeros(E * 4, E)
    balanced = torch.arange(E).repeat(4).unsqueeze(1)
    assert math.isclose(oracle.switch_aux_loss(uniform, balanced).item(), 1.0 + 0.1 * math.log(E) ** 2, rel_tol=1e-5)


def _e4m3fn_table():
    """All 256 values of OCP float8 e4m3fn from the format definition: 1-4-3 bits, bias 7, no
    infinities, S.1111.111 is NaN, exponent 0 is subnormal (2^-6 * m/8)."""
    out = []
    for b in range(256):
        s = -1.0 if b & 0x80 else 1.0
        e = (b >> 3) & 0xF
        m = b & 0x7
        if e == 0xF and m == 0x7:
            out.append(float("nan"))
        elif e == 0:
            out.append(s * (m / 8.0) * 2.0 ** -6)
        else:
            out.append(s * (1.0 + m / 8.0) * 2.0 ** (e - 7))
    return np.array(out)


def test_dequant_fp8_all_bit_patterns():
    table = _e4m3fn_table()
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).reshape(1, 1, 256)
    got = oracle.dequant_fp8(codes, torch.tensor([[0.5]]))[0, 0].double().numpy()
    finite = ~np.isnan(table)
    assert np.array_equal(np.isnan(got), ~finite)
    assert np.array_equal(got[finite], 0.5 * table[finite])
    assert np.nanmax(np.abs(table)) == 448.0


def test_quantize_fp8_per_channel_roundtrip():
    g = torch.Generator().manual_seed(18)
    w = torch.randn(3, 7, 64, generator=g) * 0.02
    q, scale = oracle.quantize_fp8_per_channel(w)
    assert q.dtype == torch.float8_e4m3fn and scale.shape == (3, 7)
    torch.testing.assert_close(scale, w.abs().amax(-1) / 448.0)
    deq = oracle.dequant_fp8(q, scale)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normal values, the row maximum is exact
    assert ((deq - w).abs() <= w.abs() * 2.0 ** -4 + scale.unsqueeze(-1) * 2.0 ** -9).all()
    assert torch.allclose(deq.abs().amax(-1), w.abs().amax(-1), rtol=1e-6)


# ---------------------------------------------------------------------------------------------------
# synthetic workloads
# ---------------------------------------------------------------------------------------------------


def test_workload_inputs_are_seeded_and_shaped():
    w = oracle.WORKLOADS["tiny-fp32"]
    a, b = oracle.make_inputs(w), oracle.make_inputs(w)
    for name in ("x", "gate_w", "w_fc", "w_proj"):
        assert torch.equal(a[name], b[name])
    assert a["x"].shape == (512, 256) and a["w_fc"].shape == (8, 1024, 256) and a["w_proj"].shape == (8, 256, 512)
    assert abs(a["x"].std().item() - 1.0) < 0.02 and abs(a["w_fc"].std().item() - 0.02) < 1e-3
    assert a["bias"] is None
    # fewer tokens: same weights
    c = oracle.make_inputs(w, T=16)
    assert torch.equal(c["w_fc"], a["w_fc"]) and c["x"].shape == (16, 256)


def test_zipf_bias_skews_the_load():
    w = oracle.WORKLOADS["granite-3b-a800m"]
    g = torch.Generator().manual_seed(w.seed)
    bias = oracle.zipf_bias(w.E, w.k, w.zipf_s, g, logit_std=0.02 * math.sqrt(w.H))
    assert bias.shape == (w.E,)
    g2 = torch.Generator().manual_seed(1)
    logits = torch.randn(20000, w.E, generator=g2) * (0.02 * math.sqrt(w.H)) + bias
    first = torch.bincount(logits.argmax(-1), minlength=w.E).double() / 20000
    ranks = torch.arange(1, w.E + 1, dtype=torch.float64).pow(-w.zipf_s)
    p_max = float(ranks[0] / ranks.sum())
    assert abs(first.max().item() - p_max) < 0.05 * p_max + 0.01  # top-1 share follows Zipf(1.1)
    load = torch.bincount(logits.topk(w.k, -1).indices.flatten(), minlength=w.E).double()
    assert load.max() / load.min() > 8  # slot counts differ by about an order of magnitude


def test_rmsnorm_equals_torch_module_and_closed_form():
    """oracle.rmsnorm is pinned by torch.nn.RMSNorm itself (the class the reference subclasses,
    normalization.py:19) bit for bit in bf16 / fp16 / fp32, and by a closed form: rows of constant magnitude c
    normalise to sign(x) * weight (up to eps)."""
    g = torch.Generator().manual_seed(2)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        x = (torch.randn(37, 96, generator=g) * 1.7).to(dtype)
        w = (1 + 0.1 * torch.randn(96, generator=g)).to(dtype)
        m = torch.nn.RMSNorm(96, eps=1e-5).to(dtype)
        with torch.no_grad():
            m.weight.copy_(w)
            want = m(x)
        assert torch.equal(oracle.rmsnorm(x, w, 1e-5), want), dtype
        assert torch.equal(oracle.rmsnorm(x, None, 1e-5), torch.nn.functional.rms_norm(x, (96,), None, 1e-5)), dtype
    s = torch.where(torch.rand(5, 64, generator=g) < 0.5, -3.0, 3.0)
    w = torch.linspace(0.5, 2.0, 64)
    torch.testing.assert_close(oracle.rmsnorm(s, w, 0.0), torch.sign(s) * w, rtol=1e-6, atol=1e-6)
