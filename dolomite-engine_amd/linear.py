"""``nn.Linear`` with N(0, std) initialisation (lm_engine/hf_models/modeling_utils/linear.py:11-33)."""

import torch
import torch.nn as nn

from .parameter import mark_parameter_as_no_weight_decay


class ParameterizedLinear(nn.Linear):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None,
                 std: float | None = None) -> None:
        self.std = std
        super().__init__(in_features, out_features, bias, device, dtype)
        mark_parameter_as_no_weight_decay(self.bias)

    @torch.no_grad()
    def reset_parameters(self) -> None:
        if self.std is None:
            super().reset_parameters()
        else:
            nn.init.normal_(self.weight, mean=0, std=self.std)
            if getattr(self, "bias", None) is not None:
                self.bias.zero_()
