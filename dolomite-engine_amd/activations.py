"""Activation registry for the MoE block.

Names and GLU semantics follow lm_engine/hf_models/modeling_utils/activations/{__init__,base,glu}.py:
a ``*glu`` activation splits its input in two halves along the last dimension and returns
``first * act(second)`` (glu.py:42-43); ``swiglu`` uses SiLU (glu.py:27, base.py:31-32).  Only
activations that exist in torch.nn are registered.
"""

import torch
import torch.nn as nn


class _ReLUSquared(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.square(torch.relu(x))


_BASE = {
    "celu": nn.CELU,
    "elu": nn.ELU,
    "gelu": nn.GELU,
    "gelu_pytorch_tanh": lambda: nn.GELU(approximate="tanh"),
    "selu": nn.SELU,
    "hard_shrink": nn.Hardshrink,
    "hard_sigmoid": nn.Hardsigmoid,
    "hard_swish": nn.Hardswish,
    "hard_tanh": nn.Hardtanh,
    "identity": nn.Identity,
    "leaky_reLU": nn.LeakyReLU,
    "log_sigmoid": nn.LogSigmoid,
    "mish": nn.Mish,
    "prelu": nn.PReLU,
    "relu": nn.ReLU,
    "relu2": _ReLUSquared,
    "relu_squared": _ReLUSquared,
    "relu6": nn.ReLU6,
    "rrelu": nn.RReLU,
    "sigmoid": nn.Sigmoid,
    "silu": nn.SiLU,
    "swish": nn.SiLU,
    "softplus": nn.Softplus,
    "soft_plus": nn.Softplus,
    "soft_shrink": nn.Softshrink,
    "soft_sign": nn.Softsign,
    "tanh": nn.Tanh,
    "tanh_shrink": nn.Tanhshrink,
}

_GLU_BASE = {
    "ceglu": "celu",
    "eglu": "elu",
    "geglu": "gelu",
    "miglu": "mish",
    "mishglu": "mish",
    "preglu": "prelu",
    "reglu": "relu",
    "rreglu": "rrelu",
    "seglu": "selu",
    "swiglu": "swish",
}


def get_base_activation(name: str) -> nn.Module:
    if name in _BASE:
        return _BASE[name]()
    raise ValueError("invalid activation function")


class GLUActivation(nn.Module):
    def __init__(self, base_activation: nn.Module) -> None:
        super().__init__()
        self.base_activation = base_activation

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        first, second = x.chunk(2, dim=-1)
        return first * self.base_activation(second)


def is_glu(name: str) -> bool:
    return name.endswith("glu")


def get_glu_activation(name: str) -> nn.Module:
    if name in ("glu", "sigmoid_glu"):
        return nn.GLU()
    if name in _GLU_BASE:
        base = _GLU_BASE[name]
    elif name.endswith("_glu"):
        base = name[: -len("_glu")]
    else:
        raise ValueError("invalid activation function")
    return GLUActivation(get_base_activation(base))


def get_activation_function(name: str | None) -> nn.Module:
    if name is None:
        return nn.Identity()
    return get_glu_activation(name) if is_glu(name) else get_base_activation(name)
