"""MoE layer with the scattered-expert forward on MI355X.

Same constructor, attributes, state-dict names/shapes and forward contract as the reference's
``MoE`` / ``ParameterizedExperts`` (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:48-384):

    gate.weight   (E, H)
    c_fc.weight   (E, 2I, H) for a GLU activation ([up ; gate] rows), else (E, I, H)
    c_proj.weight (E, H, I)
    (+ c_fc_shared / c_proj_shared when shared_intermediate_size is given)

With ``enable_kernels([Kernel.scattermoe])`` the expert computation runs on the HIP kernels of
this package (router -> sort/bin -> grouped up-projection with fused SwiGLU -> grouped
down-projection -> gate-weighted combine).  Without it the eager torch branch runs, which is the
reference's own eager branch (moe.py:292-307) and works on any device.

The kernel branch also trains: when a gradient is needed a SwiGLU layer runs its experts through
``autograd.ScatteredSwiGLUExperts``, any other activation through the differentiable ``ops.scattered_experts``
(``autograd.ScatteredExperts``), and the auxiliary loss through ``autograd.SwitchAuxLoss``.  It raises if the kernel
library is missing -- it never falls back silently.
"""

from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .activations import GLUActivation, get_activation_function, is_glu
from .autograd import FusedRouter, ScatteredSwiGLUExperts, SwitchAuxLoss, one_expert_rows
from .enums import Kernel
from .kernels import is_kernel_allowed
from .linear import ParameterizedLinear
from .loss import add_aux_loss
from .parameter import mark_parameter_as_mup_learning_rate, mark_parameter_as_no_weight_decay


def _get_std_for_linear(initializer_range: float, init_method: str, m_width: float | None) -> float:
    """lm_engine/hf_models/modeling_utils/mlp_blocks/mlp.py:58-65."""
    std = initializer_range
    if init_method == "mup":
        std /= math.sqrt(m_width)
    elif init_method != "normal":
        raise ValueError(f"unexpected init_method ({init_method})")
    return std


def bincount(x: torch.Tensor, minlength: int) -> torch.Tensor:
    """moe.py:27-30."""
    return x.bincount(minlength=minlength).to(torch.uint32)


def compute_bincount(x: torch.Tensor, size: int, use_continuous_count: bool) -> torch.Tensor:
    """moe.py:38-44: the HIP histogram when asked for, else torch.bincount."""
    if use_continuous_count:
        return ops.continuous_count(x, size=size)
    return bincount(x, minlength=size)


class ParameterizedExperts(nn.Module):
    """E stacked linear layers, weight (E, out, in) (moe.py:48-121)."""

    def __init__(self, num_experts: int, in_features: int, out_features: int, add_bias: bool = True,
                 device=None, dtype=None, std: float | None = None) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features, device=device, dtype=dtype))
        self.bias = None
        if add_bias:
            self.bias = nn.Parameter(torch.empty(num_experts, out_features, device=device, dtype=dtype))
        self.std = std
        self.num_experts = num_experts
        self.in_features = in_features
        self.out_features = out_features
        # optional fp8 storage (see MoE.quantize_expert_weights_fp8)
        self.weight_scale_dtype = None
        self.weight_q_glu = False
        self.register_buffer("weight_q", None, persistent=True)
        self.register_buffer("weight_scale", None, persistent=True)
        self.reset_parameters()
        mark_parameter_as_no_weight_decay(self.bias)

    def dense_weight(self) -> torch.Tensor:
        """The (E, out, in) weight the eager branch multiplies with (dequantised if stored as fp8)."""
        if self.weight_q is not None:
            w_q = self.weight_q
            if w_q.dim() == 1:  # streamed-tile layout
                w_q = ops.fp8_untile(w_q, self.num_experts, self.out_features, self.in_features, self.weight_q_glu)
            return (w_q.float() * self.weight_scale.unsqueeze(-1)).to(self.weight_scale_dtype)
        return self.weight

    def forward(self, input: torch.Tensor, num_experts_per_token: int | None = None,
                num_tokens_per_expert: torch.Tensor | None = None,
                sorted_expert_idxs: torch.Tensor | None = None, sorted_scattered_idxs: torch.Tensor | None = None,
                expert_offsets: torch.Tensor | None = None, gates: torch.Tensor | None = None,
                grouped_in: bool = False, grouped_out: bool = False, combine_tail: tuple | None = None) -> torch.Tensor:
        if is_kernel_allowed(Kernel.scattermoe):
            assert self.bias is None
            if self.weight_q is not None:
                raise RuntimeError("fp8 expert weights are only supported through MoE.forward")
            return ops.scattered_experts(
                inputs=input,
                expert_weights=self.weight.permute(0, 2, 1),
                k=num_experts_per_token,
                sorted_expert_idxs=sorted_expert_idxs,
                sorted_scattered_idxs=sorted_scattered_idxs,
                expert_offsets=expert_offsets,
                gates=gates,
                grouped_in=grouped_in,
                grouped_out=grouped_out,
                combine_tail=combine_tail,
            )
        weight = self.dense_weight()
        pieces = input.split(num_tokens_per_expert.tolist(), dim=0)
        outs = [
            F.linear(pieces[i], weight[i].to(input.dtype), None if self.bias is None else self.bias[i])
            for i in range(self.num_experts)
        ]
        return torch.cat(outs, dim=0)

    def extra_repr(self) -> str:
        return "num_experts={}, in_features={}, out_features={}".format(
            self.num_experts, self.in_features, self.out_features
        )

    @torch.no_grad()
    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0, std=self.std)
        if getattr(self, "bias", None) is not None:
            self.bias.zero_()

    @torch.no_grad()
    def set_fp8_weight(self, w_q: torch.Tensor, scale: torch.Tensor, compute_dtype: torch.dtype,
                       tiled: bool = False, glu: bool = False) -> None:
        """Install already quantised weights: ``w_q`` (E, out, in) e4m3fn row-major, ``scale`` (E, out) fp32."""
        if tuple(w_q.shape) != (self.num_experts, self.out_features, self.in_features) or w_q.dtype != torch.float8_e4m3fn:
            raise ValueError("w_q must be (E, out, in) torch.float8_e4m3fn")
        self.weight_scale_dtype = compute_dtype
        self.weight_q_glu = glu
        self.weight_q = ops.fp8_tile(w_q, glu) if (tiled and self.in_features % 128 == 0) else w_q
        self.weight_scale = scale.to(torch.float32)
        self.weight = None

    @torch.no_grad()
    def quantize_fp8(self, tiled: bool = False, glu: bool = False) -> None:
        """Replace the weight by e4m3fn values plus one fp32 scale per output channel
        (scale = max|row| / 448).  ``tiled`` stores the values in the layout the decode kernels stream
        (ops.fp8_tile; ``glu`` says that the rows are [up ; gate] halves); it needs in_features % 128 == 0
        and falls back to the row-major layout otherwise."""
        w = self.weight.detach().float()
        scale = w.abs().amax(dim=-1).clamp_min(1e-12) / 448.0
        self.set_fp8_weight((w / scale.unsqueeze(-1)).to(torch.float8_e4m3fn), scale, self.weight.dtype, tiled, glu)


class MoE(nn.Module):
    linear_class = ParameterizedExperts

    def __init__(self, hidden_size: int, intermediate_size: int, shared_intermediate_size: int | None,
                 num_experts: int, num_experts_per_tok: int, activation_function: str, add_bias: bool,
                 dropout: float, init_method: str, initializer_range: float, m_width: float | None,
                 num_layers: int, use_padding_free_transformer: bool) -> None:
        super().__init__()

        self.num_experts = num_experts
        self.top_k = num_experts_per_tok
        self.use_padding_free_transformer = use_padding_free_transformer
        # training on the kernel branch: keep the (slots, 2 * intermediate) pre-activation of the up-projection for
        # the backward (faster) or recompute it there (one grouped GEMM more, that much memory less)
        self.keep_preactivation = True

        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.shared_intermediate_size = shared_intermediate_size

        std = _get_std_for_linear(initializer_range, init_method, m_width)
        glu = is_glu(activation_function)

        self.gate = ParameterizedLinear(in_features=hidden_size, out_features=num_experts, bias=False, std=std)
        self.c_fc = self.linear_class(
            num_experts=num_experts,
            in_features=hidden_size,
            out_features=2 * intermediate_size if glu else intermediate_size,
            add_bias=add_bias,
            std=std,
        )
        if shared_intermediate_size is not None:
            self.c_fc_shared = ParameterizedLinear(
                in_features=hidden_size,
                out_features=2 * shared_intermediate_size if glu else shared_intermediate_size,
                bias=add_bias,
                std=std,
            )

        self.act = get_activation_function(activation_function)
        self._fused_swiglu = isinstance(self.act, GLUActivation) and isinstance(self.act.base_activation, nn.SiLU)

        std /= math.sqrt(2 * num_layers)

        self.c_proj = self.linear_class(
            num_experts=num_experts, in_features=intermediate_size, out_features=hidden_size, add_bias=add_bias,
            std=std,
        )
        if shared_intermediate_size is not None:
            self.c_proj_shared = ParameterizedLinear(
                in_features=shared_intermediate_size, out_features=hidden_size, bias=add_bias, std=std
            )

        self.dropout = nn.Identity() if dropout == 0 else nn.Dropout(dropout)

        # benchmark-input construct: an optional per-expert offset added to the router logits
        # before top-k (skews the expert load); None reproduces the reference exactly
        self.register_buffer("router_logit_bias", None, persistent=False)

        mark_parameter_as_mup_learning_rate(self.gate.weight)
        mark_parameter_as_mup_learning_rate(self.c_fc.weight)
        mark_parameter_as_mup_learning_rate(self.c_proj.weight)
        if shared_intermediate_size is not None:
            mark_parameter_as_mup_learning_rate(self.c_fc_shared.weight)
            mark_parameter_as_mup_learning_rate(self.c_proj_shared.weight)

    # ---------------------------------------------------------------------------------------------

    def forward(self, hidden_states: torch.Tensor, residual: torch.Tensor | None = None,
                residual_scale: float | None = None, pre_norm: tuple | None = None) -> torch.Tensor:
        """moe.py:212-244.  Extensions that take in the block's code around the layer
        (mixins/dense/layer.py:58-66):

        * ``pre_norm = (weight or None, eps)``: ``hidden_states`` is first RMS-normalised (the block's ``ln_2``);
          on the kernel branch the normalisation runs inside the router kernel;
        * ``residual`` / ``residual_scale``: the result is ``moe(...) * residual_scale + residual``; on the kernel
          branch they -- and the shared-expert sum -- are folded into the combine pass, with the roundings of the
          separate operations."""
        if not self.use_padding_free_transformer:
            batch_size, sequence_length, _ = hidden_states.shape

        hidden_states = hidden_states.view(-1, self.hidden_size)
        if residual is not None:
            residual = residual.reshape(-1, self.hidden_size)

        routed = None
        presorted = None
        if pre_norm is None and self._use_fused_router(hidden_states) and ops.router_fused_sort_supported(
            hidden_states, self.num_experts, self.top_k
        ):
            # small batch (decode): the router's finishing launch sorts the experts as well
            _, router_weights, selected_experts, *presorted = ops.router_fused_sort(
                hidden_states, self.gate.weight, self.top_k, bias=self.router_logit_bias
            )
            routed = (None, router_weights, selected_experts)
        if pre_norm is not None:
            norm_weight, norm_eps = pre_norm
            if self._use_fused_router(hidden_states) and ops.rmsnorm_router_fused_supported(
                hidden_states, self.num_experts, self.top_k
            ):
                hidden_states, _, router_weights, selected_experts = ops.rmsnorm_router_fused(
                    hidden_states, norm_weight, norm_eps, self.gate.weight, self.top_k, bias=self.router_logit_bias
                )
                routed = (None, router_weights, selected_experts)
            else:
                hidden_states = F.rms_norm(hidden_states, (self.hidden_size,), norm_weight, norm_eps)

        if routed is None:
            # (with a gradient the router function may hand back the expert sort as well)
            *routed, presorted = self._route(hidden_states)
        router_logits, router_weights, selected_experts = routed

        # the tail can only be folded in where nothing sits between the expert sum and it
        fuse_tail = (
            is_kernel_allowed(Kernel.scattermoe)
            and not self._needs_grad(hidden_states)
            and isinstance(self.dropout, nn.Identity)
            and (self.shared_intermediate_size is not None or residual is not None or residual_scale is not None)
        )
        if fuse_tail:
            shared = None if self.shared_intermediate_size is None else self._compute_shared_experts(hidden_states)
            hidden_states = self._compute_experts(hidden_states, router_weights, selected_experts,
                                                  tail=(shared, residual, residual_scale), presorted=presorted)
        else:
            moe_output = self._compute_experts(hidden_states, router_weights, selected_experts, presorted=presorted)
            if self.shared_intermediate_size is None:
                hidden_states = moe_output
            else:
                hidden_states = moe_output + self._compute_shared_experts(hidden_states)
            del moe_output

        if not self.use_padding_free_transformer:
            hidden_states = hidden_states.reshape(batch_size, sequence_length, self.hidden_size)

        hidden_states = self.dropout(hidden_states)

        if not fuse_tail:
            if residual_scale is not None:
                hidden_states = hidden_states * residual_scale
            if residual is not None:
                hidden_states = hidden_states + residual.reshape(hidden_states.shape)

        if not self.training:
            aux_loss = 0
        elif is_kernel_allowed(Kernel.scattermoe) and ops.aux_loss_supported(router_logits.view(-1, self.num_experts)):
            # both passes over the (T, E) logits fused (fp32 arithmetic; the eager line below rounds its
            # intermediates to the model dtype)
            aux_loss = SwitchAuxLoss.apply(router_logits.view(-1, self.num_experts), selected_experts)
        else:
            aux_loss = self._compute_switch_loss(
                logits=router_logits, probs=torch.softmax(router_logits, dim=-1), topk_idxs=selected_experts
            )
        add_aux_loss(aux_loss)

        return hidden_states

    def _needs_grad(self, hidden_states: torch.Tensor) -> bool:
        return torch.is_grad_enabled() and (
            hidden_states.requires_grad or any(p.requires_grad for p in self.parameters())
        )

    def _use_fused_router(self, hidden_states: torch.Tensor) -> bool:
        """The inference forms of the router kernel (sort or RMSNorm folded in, no logits kept)."""
        return (
            is_kernel_allowed(Kernel.scattermoe)
            and not self.training
            and not self._needs_grad(hidden_states)
            and hidden_states.is_cuda
            and ops.router_fused_supported(hidden_states, self.num_experts, self.top_k)
        )

    def _compute_routing_weights(self, hidden_states: torch.Tensor):
        """moe.py:246-257: (router_logits, router_weights, selected_experts)."""
        return self._route(hidden_states)[:3]

    def _route(self, hidden_states: torch.Tensor):
        """moe.py:246-257, plus the expert sort where the router produced it: (router_logits, router_weights,
        selected_experts, presorted or None).  On the kernel path the gate GEMM, top-k and softmax are one kernel in
        every dtype; in eval mode the (T, E) logits are never written (only the training aux loss and the backward
        read them); with a gradient the same kernel runs inside autograd.FusedRouter, whose backward is kernels
        too."""
        if (is_kernel_allowed(Kernel.scattermoe) and hidden_states.is_cuda
                and ops.router_fused_supported(hidden_states, self.num_experts, self.top_k)):
            if self._needs_grad(hidden_states):
                logits, weights, experts, *srt = FusedRouter.apply(hidden_states, self.gate.weight,
                                                                   self.router_logit_bias, self.top_k)
                return logits, weights, experts, (srt if srt[0] is not None else None)
            return (*ops.router_fused(hidden_states, self.gate.weight, self.top_k, bias=self.router_logit_bias,
                                      return_logits=self.training), None)

        router_logits = self.gate(hidden_states)
        if self.router_logit_bias is not None:
            router_logits = (router_logits.float() + self.router_logit_bias.float()).to(router_logits.dtype)

        if is_kernel_allowed(Kernel.scattermoe) and hidden_states.is_cuda:
            # shapes the router kernel does not take (more than 256 experts, a hidden size that is not a multiple
            # of 16): the logits come from torch, the selection still follows the kernel's tie rule (value
            # descending, expert index ascending) in training and in inference alike
            ops._warn_once(("router_unfused", self.num_experts, self.hidden_size, hidden_states.dtype),
                           f"MoE router with {self.num_experts} experts, hidden size {self.hidden_size}, "
                           f"{hidden_states.dtype}: not a shape of the fused router kernel; the logits are computed "
                           "by torch's linear layer")
            with torch.no_grad():
                router_weights, selected_experts = ops.router_topk_softmax(router_logits.detach(), self.top_k)
            if torch.is_grad_enabled() and router_logits.requires_grad:
                # the gradient flows through the selected logits: gather them at the kernel's indices and redo the
                # softmax over the k values in torch (same arithmetic: fp32 softmax, one rounding)
                picked = router_logits.gather(-1, selected_experts.long())
                router_weights = F.softmax(picked.float(), dim=-1).type_as(hidden_states)
        else:
            router_weights, selected_experts = self._get_topk(router_logits)
            router_weights = F.softmax(router_weights.float(), dim=-1)
            router_weights = router_weights.type_as(hidden_states)

        return router_logits, router_weights, selected_experts, None

    def _compute_experts(self, hidden_states: torch.Tensor, router_weights: torch.Tensor,
                         selected_experts: torch.Tensor, tail: tuple | None = None,
                         presorted: list | None = None) -> torch.Tensor:
        """``tail`` = (shared-expert output, residual, residual_scale) to fold into the combine (kernel branch);
        ``presorted`` = (sorted_expert_idxs, sorted_scattered_idxs, expert_offsets) when the router already
        produced them."""
        if is_kernel_allowed(Kernel.scattermoe):
            shared, residual, residual_scale = tail if tail is not None else (None, None, None)
            sorted_expert_idxs, sorted_scattered_idxs, expert_offsets = (
                presorted if presorted else ops.sort_bin(selected_experts, self.num_experts)
            )

            if self.c_fc.weight_q is None and self._fused_swiglu and self._needs_grad(hidden_states):
                # training: the same forward kernels inside a differentiable function (autograd.py)
                assert self.c_fc.bias is None and tail is None
                hidden_states = ScatteredSwiGLUExperts.apply(
                    hidden_states, self.c_fc.weight, self.c_proj.weight, router_weights, sorted_scattered_idxs,
                    expert_offsets, self.top_k, self.keep_preactivation
                )
            elif self.c_fc.weight_q is not None:
                if not self._fused_swiglu:
                    raise RuntimeError("fp8 expert weights need the swiglu activation")
                if self.hidden_size % 16 or self.intermediate_size % 16:
                    # the fp8 kernels read the weights 16 at a time: other sizes run the 16-bit kernels on weights
                    # widened for the call (round(w * scale), what the eager branch multiplies with)
                    ops._warn_once(("fp8_widened", self.hidden_size, self.intermediate_size),
                                   f"MoE with fp8 expert weights, hidden size {self.hidden_size}, intermediate size "
                                   f"{self.intermediate_size}: the fp8 kernels need multiples of 16; widening the "
                                   "weights on every call")
                    hidden_states = ops.up_swiglu(hidden_states, self.c_fc.dense_weight(), self.top_k,
                                                  sorted_scattered_idxs, expert_offsets)
                    hidden_states = ops.scattered_gemm(hidden_states, self.c_proj.dense_weight(), 1,
                                                       sorted_scattered_idxs, expert_offsets, True, False)
                else:
                    hidden_states = ops.up_swiglu_fp8(hidden_states, self.c_fc.weight_q, self.c_fc.weight_scale,
                                                      self.top_k, sorted_scattered_idxs, expert_offsets)
                    hidden_states = ops.down_fp8(hidden_states, self.c_proj.weight_q, self.c_proj.weight_scale,
                                                 sorted_scattered_idxs, expert_offsets)
                hidden_states = ops.combine(hidden_states, router_weights, shared, residual, residual_scale)
            else:
                if self._fused_swiglu:
                    assert self.c_fc.bias is None
                    hidden_states = ops.up_swiglu(hidden_states, self.c_fc.weight, self.top_k,
                                                  sorted_scattered_idxs, expert_offsets)
                else:
                    hidden_states = self.c_fc(
                        input=hidden_states,
                        num_experts_per_token=self.top_k,
                        sorted_expert_idxs=sorted_expert_idxs,
                        sorted_scattered_idxs=sorted_scattered_idxs,
                        expert_offsets=expert_offsets,
                        grouped_out=True,
                    )
                    hidden_states = self.act(hidden_states)
                hidden_states = self.c_proj(
                    input=hidden_states,
                    num_experts_per_token=1,
                    sorted_expert_idxs=sorted_expert_idxs,
                    sorted_scattered_idxs=sorted_scattered_idxs,
                    expert_offsets=expert_offsets,
                    grouped_in=True,
                    gates=router_weights,
                    combine_tail=tail,
                )
            hidden_states = self.dropout(hidden_states)
        else:
            total_q = hidden_states.shape[0]

            batch_index, batch_gates, num_tokens_per_expert = self._compute_expert_assignment(
                router_weights, selected_experts
            )

            hidden_states = hidden_states[batch_index]
            hidden_states = self.c_fc(input=hidden_states, num_tokens_per_expert=num_tokens_per_expert)
            hidden_states = self.act(hidden_states)
            hidden_states = self.c_proj(input=hidden_states, num_tokens_per_expert=num_tokens_per_expert)

            hidden_states = hidden_states * batch_gates.unsqueeze(-1)
            zeros = torch.zeros((total_q, self.hidden_size), dtype=hidden_states.dtype, device=hidden_states.device)
            hidden_states = zeros.index_add(0, batch_index, hidden_states)

        return hidden_states

    def _compute_shared_experts(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """moe.py:311-315.  On the kernel branch the dense MLP runs on the grouped-GEMM kernels as ONE expert that
        owns every token (rows in place, no gather, no router weights): SwiGLU in the up-projection's epilogue in
        inference, the differentiable forms of autograd.py when a gradient is needed; any of the three dtypes."""
        if (
            is_kernel_allowed(Kernel.scattermoe) and hidden_states.is_cuda
            and self.c_fc_shared.bias is None and self.c_proj_shared.bias is None
            and hidden_states.dtype in (torch.bfloat16, torch.float16, torch.float32)
        ):
            T = hidden_states.shape[0]
            rows, offsets = one_expert_rows(T, hidden_states.device)
            w_fc, w_proj = self.c_fc_shared.weight.unsqueeze(0), self.c_proj_shared.weight.unsqueeze(0)
            if self._fused_swiglu and self._needs_grad(hidden_states):
                return ScatteredSwiGLUExperts.apply(hidden_states, w_fc, w_proj, None, rows, offsets, 1,
                                                    self.keep_preactivation)
            if self._fused_swiglu:
                act = ops.up_swiglu(hidden_states, w_fc, 1, rows, offsets)
                return ops.scattered_gemm(act, w_proj, 1, rows, offsets, True, True)
            # any other activation: the two products through the (differentiable) drop-in op, torch in between
            kw = dict(k=1, sorted_expert_idxs=None, sorted_scattered_idxs=rows, expert_offsets=offsets,
                      grouped_in=True, grouped_out=True)
            hidden_states = ops.scattered_experts(hidden_states, w_fc.permute(0, 2, 1), **kw)
            hidden_states = self.act(hidden_states)
            return ops.scattered_experts(hidden_states, w_proj.permute(0, 2, 1), **kw)
        hidden_states = self.c_fc_shared(hidden_states)
        hidden_states = self.act(hidden_states)
        hidden_states = self.c_proj_shared(hidden_states)
        return hidden_states

    def _compute_expert_assignment(self, router_weights: torch.Tensor, selected_experts: torch.Tensor):
        """moe.py:317-336 (stable sort: within-expert order is then defined)."""
        selected_experts = selected_experts.flatten().long()
        num_tokens_per_expert = compute_bincount(
            x=selected_experts, size=self.num_experts,
            use_continuous_count=selected_experts.is_cuda and is_kernel_allowed(Kernel.continuous_count_cute),
        )
        _, index_sorted_experts = selected_experts.sort(stable=True)
        batch_index = index_sorted_experts // self.top_k
        batch_gates = router_weights.flatten()[index_sorted_experts]
        return batch_index, batch_gates, num_tokens_per_expert

    def _get_topk(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """moe.py:338-344."""
        if self.top_k == 1:
            x, indices = x.max(dim=-1, keepdim=True)
        else:
            x, indices = x.topk(self.top_k, dim=-1)
        return x, indices

    def _compute_switch_loss(self, logits: torch.Tensor, probs: torch.Tensor, topk_idxs: torch.Tensor) -> torch.Tensor:
        """moe.py:346-369 for a single data-parallel rank."""
        logits = logits.view(-1, logits.size(-1))
        probs = probs.view(-1, probs.size(-1))

        num_experts = logits.size(1)
        acc_probs = probs.sum(0)
        freq = compute_bincount(
            x=topk_idxs.flatten().long(), size=num_experts,
            use_continuous_count=topk_idxs.is_cuda and is_kernel_allowed(Kernel.continuous_count_cute),
        ).float()

        switch_loss = num_experts * (F.normalize(acc_probs, p=1, dim=0) * F.normalize(freq, p=1, dim=0)).sum()
        z_loss = (torch.logsumexp(logits, dim=-1) ** 2).mean()
        loss = switch_loss + 0.1 * z_loss
        return loss.type_as(logits)

    def get_num_active_parameters(self) -> int:
        """moe.py:371-384."""
        num_elements = 0
        for parameter in self.parameters():
            num_elements += parameter.numel()
        for parameter in self.c_fc.parameters():
            num_elements -= parameter.numel()
            num_elements += (parameter.numel() * self.top_k) // self.num_experts
        for parameter in self.c_proj.parameters():
            num_elements -= parameter.numel()
            num_elements += (parameter.numel() * self.top_k) // parameter.size(0)
        return num_elements

    @torch.no_grad()
    def quantize_expert_weights_fp8(self, tiled: bool = True) -> None:
        """Store c_fc / c_proj as e4m3fn + per-output-channel fp32 scales (decode-shape serving).
        Not part of the reference; the eager branch then multiplies with the dequantised weights.
        ``tiled`` (default) keeps the bytes in the order the decode kernels stream them (one contiguous
        run per wave); results do not depend on it."""
        if self.c_fc.bias is not None or self.c_proj.bias is not None:
            raise RuntimeError("fp8 expert weights do not support biases")
        self.c_fc.quantize_fp8(tiled=tiled, glu=self._fused_swiglu)
        self.c_proj.quantize_fp8(tiled=tiled, glu=False)
