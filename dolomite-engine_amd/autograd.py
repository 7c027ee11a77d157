"""Training through the kernel branch: the expert computation as a differentiable function.

The forward is the same three launches as in inference (up-projection with fused SwiGLU, down-projection,
combine).  The backward reuses the grouped GEMM for everything that is a "rows times expert weight" product --
the gradient w.r.t. the activations of both projections and the recomputation of the two intermediates that
are not kept -- and a second kernel, a grouped X^T dY contracted over each expert's rows, for the weight
gradients (fp32 and odd shapes run a one-thread-per-element form of it; nothing synchronises with the host).  The reference gets both from the external scattermoe autograd function
(lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:91-101); this module is the counterpart for the
gradient, built on this package's forward kernels.

Memory kept for the backward: x, the gates, the routing indices and -- by default -- the (L, 2I) pre-activation
h of the up-projection (the up-projection then writes h next to the activation and forms the activation from
the rounded h, as the reference's grouped GEMM followed by GLUActivation does, moe.py:273-281; shapes the tile
kernel does not take run exactly those two steps); with ``keep_preactivation=False`` h is recomputed
in the backward from x and the forward keeps its fused up-projection (one more grouped GEMM per step, L * 2I
elements less memory).  The (L, I) activation follows from h, and the (L, H) expert outputs are never needed (the
gradient of a router weight, <dy[t], w_proj[e] a>, is taken as <w_proj[e]^T dy[t], a>).
"""

from __future__ import annotations

import torch

from . import ops


class ScatteredSwiGLUExperts(torch.autograd.Function):
    """y[t] = sum_j gates[t, j] * ( swiglu(x[t] @ w_fc[e]^T) @ w_proj[e]^T ),  e = expert of slot (t, j).

    ``gates=None`` (needs k == 1): no router weights and no combine pass, y is the rows of the down-projection in
    flat-slot order -- the shared experts (moe.py:311-315) run this way as one expert that owns every token."""

    @staticmethod
    def forward(ctx, x, w_fc, w_proj, gates, sorted_scattered, expert_offsets, k, keep_preactivation=True):
        h = None
        if keep_preactivation:
            act, h = ops.up_swiglu_keep(x, w_fc, k, sorted_scattered, expert_offsets)
        else:
            act = ops.up_swiglu(x, w_fc, k, sorted_scattered, expert_offsets)
        o = ops.scattered_gemm(act, w_proj, 1, sorted_scattered, expert_offsets, True, False)
        if gates is None:
            if k != 1:
                raise ValueError("gates=None needs k == 1")
            y = o
        else:
            y = ops.combine(o, gates)
        ctx.save_for_backward(x, w_fc, w_proj, gates, sorted_scattered, expert_offsets, h)
        ctx.k = k
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w_fc, w_proj, gates, ss, off, h = ctx.saved_tensors
        k = ctx.k
        T, H = x.shape
        E, I2, _ = w_fc.shape
        I = I2 // 2
        dy = dy.contiguous()
        half = ops.elementwise_supported(x.dtype, I)  # (else: a ragged intermediate size, torch arithmetic)

        # gradient w.r.t. the SwiGLU output a, in sorted order and before the router weight: dy[t_i] @ w_proj[e_i]
        d_act = ops.scattered_gemm(dy, w_proj, k, ss, off, False, True, weight_kn=True)
        # pre-activation kept or recomputed; one pass then gives d_h (with the router weight g_i of the row applied),
        # g_i * a_i for the down-projection's weight gradient, and the gradient of the router weights,
        # <dy[t], w_proj[e] a_i> = <d_act_i, a_i>
        if h is None:
            h = ops.scattered_gemm(x, w_fc, k, ss, off, False, True)
        if half:
            d_h, act_g, d_gates = ops.swiglu_backward(h, d_act, gates, ss if gates is not None else None,
                                                      want_act=True, want_gate_grad=gates is not None)
        else:
            ssl = ss.long()
            up, gate, da = h[:, :I].float(), h[:, I:].float(), d_act.float()
            sig = torch.sigmoid(gate)
            a = up * gate * sig
            if gates is None:
                g_sorted, d_gates = 1.0, None
            else:
                g_sorted = gates.reshape(-1)[ssl].float().unsqueeze(-1)
                d_gates = torch.empty(T * k, dtype=torch.float32, device=x.device)
                d_gates[ssl] = (da * a).sum(dim=1)
                d_gates = d_gates.view(T, k).to(gates.dtype)
            da = da * g_sorted
            d_h = torch.cat([da * gate * sig, da * up * sig * (1.0 + gate * (1.0 - sig))], dim=1).to(x.dtype)
            act_g = (a * g_sorted).to(x.dtype)
            del up, gate, sig, da, a
        del h, d_act

        # gradient w.r.t. x: every slot's contribution in flat-slot order, then the k slots of a token summed
        dx_slots = ops.scattered_gemm(d_h, w_fc, 1, ss, off, True, False, weight_kn=True)
        # (the k slots of a token summed in slot order by the combine kernel with unit gates)
        dx = dx_slots if k == 1 else ops.combine(dx_slots, _unit_gates(T, k, x.dtype, x.device))
        del dx_slots

        # weight gradients: per expert X^T dY over that expert's rows
        tok32 = torch.div(ss, k, rounding_mode="floor").to(torch.int32)
        d_w_fc = ops.grouped_wgrad(d_h, x, off, None, tok32)
        d_w_proj = ops.grouped_wgrad(dy, act_g, off, tok32, None)
        return dx, d_w_fc, d_w_proj, d_gates, None, None, None, None


class ScatteredExperts(torch.autograd.Function):
    """One grouped GEMM of the layer with a gradient: the differentiable form of ``ops.scattered_experts``
    (the reference's external op is differentiable too, moe.py:91-101), for expert MLPs whose activation is not the
    fused SwiGLU.

        out[orow(i)] = x[irow(i)] @ w[e_i]^T           i = sorted row, w (E, N, K)
        irow(i) = i (grouped_in) or sorted_scattered[i] // k;   orow(i) = i (grouped_out) or sorted_scattered[i]
        with gates (T, kg):  y[t] = sum_j gates[t, j] * out[t * kg + j]

    Backward: d x from the transposed-weight form of the same kernel, d w from the grouped weight-gradient kernel
    (matrix cores for 16-bit dtypes, a one-thread-per-element kernel otherwise), d gates from the recomputed rows."""

    @staticmethod
    def forward(ctx, x, w, k, sorted_scattered, expert_offsets, gates, grouped_in, grouped_out):
        out = ops.scattered_gemm(x, w, k, sorted_scattered, expert_offsets, grouped_in, grouped_out)
        if gates is not None:
            out = ops.combine(out, gates.to(out.dtype))
        ctx.save_for_backward(x, w, sorted_scattered, expert_offsets, gates)
        ctx.cfg = (k, grouped_in, grouped_out)
        return out

    @staticmethod
    def backward(ctx, d_out):
        x, w, ss, off, gates = ctx.saved_tensors
        k, grouped_in, grouped_out = ctx.cfg
        E, N, K = w.shape
        L = ss.numel()
        d_out = d_out.contiguous()
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]

        d_gates = None
        if gates is not None:
            T, kg = gates.shape
            if ctx.needs_input_grad[5]:
                rows = ops.scattered_gemm(x, w, k, ss, off, grouped_in, False)
                if ops.elementwise_supported(rows.dtype, N):
                    d_gates = ops.combine_grad_gates(rows, d_out, kg).to(gates.dtype)
                else:
                    d_gates = torch.bmm(rows.view(T, kg, N), d_out.unsqueeze(-1)).squeeze(-1).to(gates.dtype)
                del rows
            # gradient of the (L, N) rows in flat-slot order
            d_out = (gates.to(d_out.dtype).unsqueeze(-1) * d_out.unsqueeze(1)).reshape(L, N)

        dx = None
        if need_x:
            # row i: d_out[orow(i)] @ w[e_i], delivered to irow(i) (kept per slot first when a token fans out to k)
            dx = ops.scattered_gemm(d_out, w, 1, ss, off, grouped_out, grouped_in, weight_kn=True)
            if not grouped_in and k > 1:
                dx = ops.combine(dx, _unit_gates(L // k, k, dx.dtype, dx.device))

        dw = None
        if need_w:
            a_idx = None if grouped_out else ss.to(torch.int32)
            b_idx = None if grouped_in else torch.div(ss, k, rounding_mode="floor").to(torch.int32)
            dw = ops.grouped_wgrad(d_out, x, off, a_idx, b_idx)
        return dx, dw, None, None, None, d_gates, None, None


class SwitchAuxLoss(torch.autograd.Function):
    """The router's auxiliary loss (moe.py:346-369, one data-parallel rank) as two fused passes over the logits:
    value in the forward, gradient w.r.t. the logits in the backward.  Returns a 0-d tensor in the logits' dtype."""

    @staticmethod
    def forward(ctx, logits, topk_idxs):
        loss_w = ops.aux_loss(logits.detach(), topk_idxs)
        ctx.save_for_backward(logits, loss_w)
        return loss_w[0].to(logits.dtype)

    @staticmethod
    def backward(ctx, grad):
        logits, loss_w = ctx.saved_tensors
        return ops.aux_loss_backward(logits.detach(), loss_w, grad), None


_ONE_EXPERT_ROWS: dict = {}
_ONE_EXPERT_ROWS_MAX = 16
_UNIT_GATES: dict = {}


def _unit_gates(T: int, k: int, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """(T, k) ones: the gates with which the combine kernel adds a token's k slots in slot order.  Read-only and
    kept per shape like :func:`one_expert_rows` (never released; made per call beyond a few shapes)."""
    key = (T, k, dtype, device.index)
    hit = _UNIT_GATES.get(key)
    if hit is None:
        hit = torch.ones((T, k), dtype=dtype, device=device)
        if len(_UNIT_GATES) < _ONE_EXPERT_ROWS_MAX and not _capturing():
            _UNIT_GATES[key] = hit
    return hit


def _capturing() -> bool:
    """A tensor filled while a graph is being captured holds its values only once the graph has run: such tensors
    are not kept for later calls."""
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def one_expert_rows(T: int, device: torch.device):
    """(sorted_scattered_idxs, expert_offsets) of one expert that owns rows 0..T-1 in order.  Read-only and kept per
    (T, device) -- never released, so a captured graph may hold their addresses; beyond a few shapes they are made
    per call."""
    key = (T, device.index)
    hit = _ONE_EXPERT_ROWS.get(key)
    if hit is not None:
        return hit
    made = (torch.arange(T, dtype=torch.int32, device=device), torch.full((1,), T, dtype=torch.int32, device=device))
    if len(_ONE_EXPERT_ROWS) < _ONE_EXPERT_ROWS_MAX and not _capturing():
        _ONE_EXPERT_ROWS[key] = made
    return made


class FusedRouter(torch.autograd.Function):
    """MoE._compute_routing_weights (moe.py:246-257) as one differentiable function on this package's kernels:

        logits = x @ gate_w^T (+ bias) in x.dtype;  experts = top-k;  gates = softmax over the k picked logits

    Returns (logits, gates, experts, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets); the last three are
    the expert sort of the selection where the router kernel can fold it in (ops.router_fused_sort: its first pass
    is the router's epilogue), else None and the caller sorts.  The backward takes the gradients that arrive at
    ``gates`` (from the expert combine) and at ``logits`` (from the auxiliary loss), forms d logits in one
    element-wise kernel and runs the two products d x = d logits @ gate_w and d gate_w = d logits^T @ x on the
    grouped GEMM / grouped weight-gradient kernels as one expert that owns every token: no library GEMM in either
    direction."""

    @staticmethod
    def forward(ctx, x, gate_w, bias, k):
        se = ss = off = None
        if ops.router_fused_sort_supported(x, gate_w.shape[0], k):
            logits, gates, experts, se, ss, off = ops.router_fused_sort(x, gate_w, k, bias=bias, return_logits=True)
            ctx.mark_non_differentiable(experts, se, ss, off)
        else:
            logits, gates, experts = ops.router_fused(x, gate_w, k, bias=bias, return_logits=True)
            ctx.mark_non_differentiable(experts)
        ctx.save_for_backward(x, gate_w, logits, experts)
        return logits, gates, experts, se, ss, off

    @staticmethod
    def backward(ctx, d_logits, d_gates, *_):
        x, gate_w, logits, experts = ctx.saved_tensors
        T, H = x.shape
        if d_logits is None and d_gates is None:
            return None, None, None, None
        dl = ops.router_dlogits(logits, experts, d_gates, d_logits)
        rows, off = one_expert_rows(T, x.device)
        dx = dw = None
        if ctx.needs_input_grad[0]:
            # (T, E) @ (E, H): the gate weight transposed to (H, E) is the "(out, in)" weight of one expert
            dx = ops.scattered_gemm(dl, gate_w.t().contiguous().unsqueeze(0), 1, rows, off, True, True)
        if ctx.needs_input_grad[1]:
            dw = ops.grouped_wgrad(dl, x, off)[0]
        return dx, dw, None, None
