"""MI355X-native scattered-MoE forward for lm_engine (IBM/dolomite-engine).

Public surface (mirrors the reference names for this path):

* ``MoE``, ``ParameterizedExperts``            -- the layer (lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py)
* ``Kernel``, ``enable_kernels``, ``is_kernel_allowed`` -- the kernel toggle (lm_engine/kernels.py, enums.py)
* ``ops.scattered_experts``, ``ops.continuous_count``   -- stand-ins for the two external ops the reference imports
* ``add_aux_loss`` / ``get_aux_loss`` / ``clear_aux_loss`` -- the aux-loss side channel
"""

from . import ops
from ._lib import MiMoeError, build, is_built
from .activations import get_activation_function, is_glu
from .enums import Kernel
from .kernels import enable_all_kernels, enable_kernels, is_kernel_allowed
from .linear import ParameterizedLinear
from .loss import add_aux_loss, clear_aux_loss, get_aux_loss, is_aux_loss_zero
from .moe import MoE, ParameterizedExperts, compute_bincount

__all__ = [
    "MoE", "ParameterizedExperts", "ParameterizedLinear", "Kernel", "enable_kernels", "enable_all_kernels",
    "is_kernel_allowed", "ops", "build", "is_built", "MiMoeError", "add_aux_loss", "clear_aux_loss",
    "get_aux_loss", "is_aux_loss_zero", "get_activation_function", "is_glu", "compute_bincount",
]
