"""Kernel switch names.

Same member names and values as the reference's ``Kernel`` enum (lm_engine/enums.py:70-89) so that
configuration files and ``enable_kernels([...])`` call sites carry over unchanged.  Only
``scattermoe`` and ``continuous_count_cute`` select code in this package; the other members exist
so that a kernel list written for the reference still parses.
"""

from enum import Enum


class Kernel(Enum):
    causal_conv1d = "causal_conv1d"
    continuous_count_cute = "continuous_count_cute"
    cross_entropy_cute = "cross_entropy_cute"
    fused_linear_cross_entropy_cute = "fused_linear_cross_entropy_cute"
    gru_cute = "gru_cute"
    pack_sequence_cute = "pack_sequence_cute"
    rmsnorm_cute = "rmsnorm_cute"
    rmsnorm_memory_efficient_cute = "rmsnorm_memory_efficient_cute"
    rnn_cute = "rnn_cute"
    swiglu_packed_cute = "swiglu_packed_cute"
    unpack_sequence_cute = "unpack_sequence_cute"
    flash_attention_2 = "flash_attention_2"
    flash_attention_3 = "flash_attention_3"
    mamba2_ssm = "mamba2_ssm"
    scattermoe = "scattermoe"
    ladder_residual_overlapped_layer = "ladder_residual_overlapped_layer"
