"""CPU oracle for the scattered-MoE layer forward.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU with plain torch ops, the arithmetic of the reference's
eager MoE branch.  It is the checker for the HIP path: only the test-suite, the smoke
entry and the benchmark's ``cpu_baseline`` leg may import it.  The product package never
imports it and has no CPU fallback for the kernel branch.

Reference files followed (paths relative to the reference tree):

* router            lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:246-257
* top-k             lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:338-344
* expert assignment lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:317-336
* sort / bin        lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:263-271 and 27-44
* per-expert linear lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:102-108
* gate + index_add  lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:292-307
* SwiGLU            lm_engine/hf_models/modeling_utils/activations/glu.py:42-43 (x[0] * silu(x[1]),
                    c_fc rows are [up ; gate], mlp_blocks/mlp.py:68-69)
* switch aux loss   lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:346-369

Two implementation-defined behaviours of the reference are fixed here by an explicit rule,
because ``torch.topk`` documents no tie order and ``Tensor.sort`` is unstable by default:

* top-k ties: larger value first, then smaller expert index first;
* expert sort: stable (slots of one expert stay in ascending flat-slot order).

The fp8 weight variant (e4m3fn weights, one fp32 scale per output channel) has no
counterpart in the reference; its oracle is "dequantise, then the fp32 path".

Pinning status (what checks each function; see tests/test_oracle_pins.py):

* router_logits        closed form GEMM vs float64 numpy
* topk_canonical       brute-force python selection on small cases; agrees with torch.topk
                       on tie-free rows
* softmax_topk         closed form in float64; invariants (sum 1, monotone)
* sort_bin             numpy stable argsort; permutation / monotonic / cumsum invariants
* experts_eager        E=1 reduces to a dense SwiGLU MLP; one-hot weights give a permuted
                       input; float64 einsum brute force; independent implementation in
                       transformers (GraniteMoe) with [gate;up] layout
* combine              brute-force loops
* switch_aux_loss      float64 restatement of the formula from its definition on tiny inputs
* dequant_fp8          exhaustive over all 256 e4m3fn bit patterns against a table built
                       from the format definition
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------
# routing
# --------------------------------------------------------------------------------------


def router_logits(x: torch.Tensor, gate_weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``gate(x)`` of moe.py:248: a bias-free linear whose result is in the model dtype.

    The product is accumulated in fp32 from the (already rounded) inputs and rounded once
    to the model dtype, which is what a library GEMM with fp32 accumulation does.  ``bias``
    is a benchmark-input construct (a per-expert logit offset that skews the load); it is
    added in fp32 to the rounded logits and the sum is rounded to the model dtype again.
    """
    dtype = x.dtype
    logits = (x.float() @ gate_weight.float().t()).to(dtype)
    if bias is not None:
        logits = (logits.float() + bias.float()).to(dtype)
    return logits


def topk_canonical(logits: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Top-k of moe.py:338-344 with the tie rule "value descending, expert index ascending".

    A stable descending sort leaves equal values in their original (ascending index) order,
    so its first k columns are exactly that rule.  For k == 1 this is ``max`` = first
    occurrence, as in moe.py:339-340.  NaN sorts as the largest value, as in torch.
    """
    vals, idx = torch.sort(logits.float(), dim=-1, descending=True, stable=True)
    return vals[:, :k].to(logits.dtype).contiguous(), idx[:, :k].contiguous()


def softmax_topk(topk_vals: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """fp32 softmax over the k selected logits, cast to the model dtype (moe.py:252-255)."""
    return F.softmax(topk_vals.float(), dim=-1).to(out_dtype)


def route(x: torch.Tensor, gate_weight: torch.Tensor, k: int, bias: torch.Tensor | None = None,
          logits: torch.Tensor | None = None):
    """moe.py:246-257.  Returns (logits, gates (T,k) model dtype, experts (T,k) int64).

    ``logits`` may be supplied (e.g. the ones a device GEMM produced) so that two routings
    are compared on identical inputs; otherwise they are computed here.
    """
    if logits is None:
        logits = router_logits(x, gate_weight, bias)
    vals, idx = topk_canonical(logits, k)
    gates = softmax_topk(vals, x.dtype)
    return logits, gates, idx


def sort_bin(selected_experts: torch.Tensor, num_experts: int):
    """moe.py:263-271: sort the flat (T*k,) expert ids, histogram them, inclusive prefix sum.

    Returns (sorted_expert_idxs, sorted_scattered_idxs, expert_offsets), all int64.  Expert e
    owns sorted rows [offsets[e-1], offsets[e]) and offsets[E-1] == T*k.
    """
    flat = selected_experts.flatten()
    sorted_expert_idxs, sorted_scattered_idxs = torch.sort(flat, stable=True)
    counts = torch.bincount(flat, minlength=num_experts)
    expert_offsets = counts.cumsum(-1)
    return sorted_expert_idxs, sorted_scattered_idxs, expert_offsets


def expert_assignment(gates: torch.Tensor, selected_experts: torch.Tensor, num_experts: int):
    """moe.py:317-336: (batch_index, batch_gates, num_tokens_per_expert) of the eager branch."""
    k = selected_experts.shape[1]
    flat = selected_experts.flatten()
    num_tokens_per_expert = torch.bincount(flat, minlength=num_experts)
    _, index_sorted = torch.sort(flat, stable=True)
    batch_index = index_sorted // k
    batch_gates = gates.flatten()[index_sorted]
    return batch_index, batch_gates, num_tokens_per_expert


# --------------------------------------------------------------------------------------
# experts
# --------------------------------------------------------------------------------------


def swiglu(h: torch.Tensor) -> torch.Tensor:
    """glu.py:42-43 with SiLU: first half is "up", second half goes through the activation."""
    up, gate = h.chunk(2, dim=-1)
    return up * F.silu(gate)


def grouped_linear(x_grouped: torch.Tensor, weight: torch.Tensor, num_tokens_per_expert: torch.Tensor) -> torch.Tensor:
    """moe.py:102-108: split rows by expert, one F.linear per expert, concatenate."""
    counts = num_tokens_per_expert.tolist()
    pieces = x_grouped.split(counts, dim=0)
    outs = [F.linear(pieces[e], weight[e]) for e in range(weight.shape[0])]
    return torch.cat(outs, dim=0)


def experts_eager(x: torch.Tensor, gates: torch.Tensor, selected_experts: torch.Tensor,
                  w_fc: torch.Tensor, w_proj: torch.Tensor, activation=swiglu,
                  compute_dtype: torch.dtype | None = torch.float32) -> torch.Tensor:
    """Eager branch of moe.py:292-307.

    ``compute_dtype=torch.float32`` (default) evaluates everything in fp32 from the given
    (already rounded) tensors: this is the acceptance oracle.  ``compute_dtype=None`` keeps
    every intermediate in the dtype of ``x`` like the reference module does.
    """
    E = w_fc.shape[0]
    T, H = x.shape
    if compute_dtype is not None:
        x, gates, w_fc, w_proj = (t.to(compute_dtype) for t in (x, gates, w_fc, w_proj))
    batch_index, batch_gates, counts = expert_assignment(gates, selected_experts, E)
    h = x[batch_index]
    h = grouped_linear(h, w_fc, counts)
    h = activation(h)
    h = grouped_linear(h, w_proj, counts)
    h = h * batch_gates.unsqueeze(-1)
    out = torch.zeros((T, H), dtype=h.dtype)
    return out.index_add(0, batch_index, h)


def scattered_experts_oracle(inputs: torch.Tensor, weight: torch.Tensor, k: int,
                             sorted_expert_idxs: torch.Tensor, sorted_scattered_idxs: torch.Tensor,
                             expert_offsets: torch.Tensor, gates: torch.Tensor | None = None,
                             grouped_in: bool = False, grouped_out: bool = False) -> torch.Tensor:
    """Semantics of the external ``scattered_experts`` call as used at moe.py:91-101, in fp32.

    ``weight`` is in the module's native (E, out, in) layout.  Row i of the sorted order uses
    expert ``sorted_expert_idxs[i]``; its input is row i (grouped_in) or row
    ``sorted_scattered_idxs[i] // k`` of ``inputs``; its output lands at row i (grouped_out) or
    row ``sorted_scattered_idxs[i]``.  With ``gates`` (T, k_g) the (L, out) result is viewed as
    (T, k_g, out) and contracted with the gates.
    """
    L = sorted_expert_idxs.numel()
    xin = inputs.float()
    rows = xin if grouped_in else xin[sorted_scattered_idxs // k]
    out = torch.empty((L, weight.shape[1]), dtype=torch.float32)
    start = 0
    for e in range(weight.shape[0]):
        end = int(expert_offsets[e])
        if end > start:
            out[start:end] = rows[start:end] @ weight[e].float().t()
        start = end
    if not grouped_out:
        scattered = torch.empty_like(out)
        scattered[sorted_scattered_idxs] = out
        out = scattered
    if gates is not None:
        kg = gates.shape[1]
        out = torch.einsum("tk,tkh->th", gates.float(), out.view(-1, kg, out.shape[-1]))
    return out


def dequant_fp8(w_q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """e4m3fn weights (E, out, in) times one fp32 scale per output channel (E, out) -> fp32."""
    return w_q.float() * scale.float().unsqueeze(-1)


def quantize_fp8_per_channel(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """scale = max|row| / 448 ; w_q = round_to_e4m3fn(w / scale).  Benchmark-input construct."""
    amax = w.float().abs().amax(dim=-1).clamp_min(1e-12)
    scale = amax / 448.0
    w_q = (w.float() / scale.unsqueeze(-1)).to(torch.float8_e4m3fn)
    return w_q, scale


# --------------------------------------------------------------------------------------
# whole layer
# --------------------------------------------------------------------------------------


@dataclass
class OracleOutput:
    y: torch.Tensor               # (T, H) fp32 (or model dtype with compute_dtype=None)
    logits: torch.Tensor          # (T, E) model dtype
    gates: torch.Tensor           # (T, k) model dtype
    experts: torch.Tensor         # (T, k) int64
    sorted_expert_idxs: torch.Tensor
    sorted_scattered_idxs: torch.Tensor
    expert_offsets: torch.Tensor


def moe_forward(x: torch.Tensor, gate_weight: torch.Tensor, w_fc: torch.Tensor, w_proj: torch.Tensor, k: int,
                bias: torch.Tensor | None = None, logits: torch.Tensor | None = None,
                w_fc_scale: torch.Tensor | None = None, w_proj_scale: torch.Tensor | None = None,
                compute_dtype: torch.dtype | None = torch.float32,
                shared_fc: torch.Tensor | None = None, shared_proj: torch.Tensor | None = None,
                residual: torch.Tensor | None = None, residual_scale: float | None = None) -> OracleOutput:
    """moe.py:212-244 in eval mode with the eager expert branch; x is (T, H).  With ``residual`` /
    ``residual_scale`` also the two lines the transformer block runs after the layer
    (mixins/dense/layer.py:61-66): y * m_residual + residual."""
    E = w_fc.shape[0]
    logits, gates, experts = route(x, gate_weight, k, bias=bias, logits=logits)
    if w_fc_scale is not None:
        w_fc = dequant_fp8(w_fc, w_fc_scale)
    if w_proj_scale is not None:
        w_proj = dequant_fp8(w_proj, w_proj_scale)
    y = experts_eager(x, gates, experts, w_fc, w_proj, compute_dtype=compute_dtype)
    if shared_fc is not None:
        xs = x if compute_dtype is None else x.to(compute_dtype)
        sf = shared_fc if compute_dtype is None else shared_fc.to(compute_dtype)
        sp = shared_proj if compute_dtype is None else shared_proj.to(compute_dtype)
        y = y + F.linear(swiglu(F.linear(xs, sf)), sp)
    if residual_scale is not None:  # mixins/dense/layer.py:61-62
        y = y * residual_scale
    if residual is not None:        # mixins/dense/layer.py:64
        y = y + (residual if compute_dtype is None else residual.to(compute_dtype))
    se, ss, off = sort_bin(experts, E)
    return OracleOutput(y, logits, gates, experts, se, ss, off)


def rmsnorm(h: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    """torch.nn.RMSNorm as the reference's RMSNorm falls back to (normalization.py:19-34): fp32 arithmetic,
    x * rsqrt(mean(x^2) + eps) * weight, one rounding to the input dtype."""
    hf = h.float()
    y = hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight.float()
    return y.to(h.dtype)


def switch_aux_loss(logits: torch.Tensor, selected_experts: torch.Tensor) -> torch.Tensor:
    """moe.py:346-369 without the data-parallel all-reduce (single process)."""
    logits = logits.view(-1, logits.size(-1))
    E = logits.size(1)
    probs = torch.softmax(logits, dim=-1)
    acc_probs = probs.sum(0)
    freq = torch.bincount(selected_experts.flatten(), minlength=E).float()
    switch = E * (F.normalize(acc_probs, p=1, dim=0) * F.normalize(freq, p=1, dim=0)).sum()
    z = (torch.logsumexp(logits, dim=-1) ** 2).mean()
    return (switch + 0.1 * z).type_as(logits)


# --------------------------------------------------------------------------------------
# seeded synthetic workloads (the five benchmark / parity configurations)
# --------------------------------------------------------------------------------------


@dataclass
class Workload:
    name: str
    T: int
    H: int
    E: int
    k: int
    I: int
    dtype: torch.dtype
    seed: int
    zipf_s: float | None = None
    fp8: bool = False


WORKLOADS = {
    "tiny-fp32": Workload("tiny-fp32", 512, 256, 8, 2, 512, torch.float32, 1235),
    "granite-1b-a400m": Workload("granite-1b-a400m", 16384, 1024, 32, 8, 512, torch.bfloat16, 1236),
    "granite-3b-a800m": Workload("granite-3b-a800m", 32768, 1536, 40, 8, 512, torch.bfloat16, 1237, zipf_s=1.1),
    "mixtral": Workload("mixtral", 8192, 4096, 8, 2, 14336, torch.bfloat16, 1238),
    "decode-fp8": Workload("decode-fp8", 64, 4096, 64, 6, 1408, torch.bfloat16, 1239, fp8=True),
}


def zipf_bias(E: int, k: int, s: float, gen: torch.Generator, logit_std: float, trials: int = 8192) -> torch.Tensor:
    """Per-expert logit offset b_e = alpha * ln p_e with p_e ~ rank^-s over a seeded permutation.

    alpha is found by bisection on a seeded sample of N(0, logit_std^2) logits so that the share of
    tokens whose FIRST choice is the most popular expert equals the Zipf probability p_max.  (The
    share of all T*k slots cannot follow Zipf itself: one expert gets at most 1/k of the slots, which
    is below p_max for k = 8.)  The realised per-expert slot counts are skewed by more than 10x.
    """
    ranks = torch.arange(1, E + 1, dtype=torch.float64)
    p = ranks.pow(-s)
    p = p / p.sum()
    perm = torch.randperm(E, generator=gen)
    logp = torch.empty(E, dtype=torch.float64)
    logp[perm] = p.log()
    target = float(p.max())
    sample = torch.randn(trials, E, generator=gen, dtype=torch.float64) * logit_std

    def first_choice_share(alpha: float) -> float:
        first = (sample + alpha * logp).argmax(dim=-1)
        return float(torch.bincount(first, minlength=E).max()) / trials

    lo, hi = 0.0, 8.0
    for _ in range(40):
        mid = 0.5 * (lo + hi)
        if first_choice_share(mid) < target:
            lo = mid
        else:
            hi = mid
    alpha = 0.5 * (lo + hi)
    return (alpha * logp).float()


def make_inputs(w: Workload, T: int | None = None) -> dict:
    """Seeded tensors of one workload: x ~ N(0,1), all weights ~ N(0, 0.02^2), drawn in fp32 on a
    CPU generator and then cast.  ``T`` overrides the token count (same weights, fewer rows)."""
    g = torch.Generator(device="cpu").manual_seed(w.seed)
    T = w.T if T is None else T
    gate_w = (torch.randn(w.E, w.H, generator=g) * 0.02).to(w.dtype)
    bias = None
    if w.zipf_s is not None:
        logit_std = 0.02 * math.sqrt(w.H)
        bias = zipf_bias(w.E, w.k, w.zipf_s, g, logit_std)
    w_fc = torch.empty(w.E, 2 * w.I, w.H, dtype=w.dtype)
    w_proj = torch.empty(w.E, w.H, w.I, dtype=w.dtype)
    fc_scale = proj_scale = None
    if w.fp8:
        w_fc = torch.empty(w.E, 2 * w.I, w.H, dtype=torch.float8_e4m3fn)
        w_proj = torch.empty(w.E, w.H, w.I, dtype=torch.float8_e4m3fn)
        fc_scale = torch.empty(w.E, 2 * w.I)
        proj_scale = torch.empty(w.E, w.H)
    for e in range(w.E):  # one expert at a time keeps the fp32 staging small
        a = torch.randn(2 * w.I, w.H, generator=g) * 0.02
        b = torch.randn(w.H, w.I, generator=g) * 0.02
        if w.fp8:
            w_fc[e], fc_scale[e] = quantize_fp8_per_channel(a)
            w_proj[e], proj_scale[e] = quantize_fp8_per_channel(b)
        else:
            w_fc[e] = a.to(w.dtype)
            w_proj[e] = b.to(w.dtype)
    x = torch.randn(T, w.H, generator=g).to(w.dtype)
    return dict(x=x, gate_w=gate_w, w_fc=w_fc, w_proj=w_proj, bias=bias, fc_scale=fc_scale, proj_scale=proj_scale)
