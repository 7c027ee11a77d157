"""CPU-side checks of the drop-in boundary: the C ABI (symbols, argument validation, error text), the
module interface (constructor, parameter names / shapes, toggle semantics) and the eager branch, which
must equal the oracle.  No kernel is launched here."""

import ctypes
import math
import os
import re

import pytest
import torch

import dolomite_engine_amd as pkg
from dolomite_engine_amd import Kernel, MoE, ParameterizedExperts, enable_kernels, is_kernel_allowed
from dolomite_engine_amd import _lib
from oracle import moe_oracle as oracle

HEADER = _lib.HEADER_PATH


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_moe_[a-z0-9_]+)\s*\(", text)))


def _moe(**kw):
    args = dict(hidden_size=32, intermediate_size=48, shared_intermediate_size=None, num_experts=8,
                num_experts_per_tok=2, activation_function="swiglu", add_bias=False, dropout=0.0,
                init_method="normal", initializer_range=0.02, m_width=None, num_layers=2,
                use_padding_free_transformer=False)
    args.update(kw)
    return MoE(**args)


# ---------------------------------------------------------------------------------------------------
# C ABI
# ---------------------------------------------------------------------------------------------------


def test_library_is_built_and_exports_every_declared_symbol():
    assert pkg.is_built(), "build the library first: python -c 'import __graft_entry__ as g; g.build()'"
    declared = _declared_functions()
    assert len(declared) >= 14
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/mi_moe.h but not exported"
    # the Python binding table covers exactly the header
    assert sorted(_lib.SIGNATURES) == declared


def test_abi_version_and_error_text():
    lib = _lib.load()
    assert lib.mi_moe_abi_version() == _lib.ABI_VERSION
    header = open(HEADER).read()
    assert f"#define MI_MOE_ABI_VERSION {_lib.ABI_VERSION}" in header
    for code, word in [(0, "ok"), (-1, "NULL"), (-2, "dimension"), (-3, "element type"), (-4, "aligned"),
                       (-5, "workspace"), (-6, "not supported"), (-7, "scratch")]:
        assert word in lib.mi_moe_strerror(code).decode()
    assert "unknown" in lib.mi_moe_strerror(-99).decode()


def test_argument_validation_happens_before_any_launch():
    """Bad shapes / NULL pointers / unsupported dtypes are refused on the host (no GPU needed)."""
    lib = _lib.load()
    E_NULL, E_SHAPE, E_DTYPE, E_WS, E_UNSUP = -1, -2, -3, -5, -6
    assert lib.mi_moe_router_topk_softmax(None, 4, 0, 1, _lib.BF16, None, None, None) == E_SHAPE
    assert lib.mi_moe_router_topk_softmax(None, 4, 8, 9, _lib.BF16, None, None, None) == E_SHAPE  # k > E
    assert lib.mi_moe_router_topk_softmax(None, 4, 8, 2, _lib.BF16, None, None, None) == E_NULL
    assert lib.mi_moe_router_topk_softmax(None, 0, 8, 2, _lib.BF16, None, None, None) == 0  # empty input
    # fp32 and up to 256 experts are taken (general kernel); beyond that, or a ragged hidden size: refused
    assert lib.mi_moe_router_fused(None, None, None, 4, 64, 128, 2, _lib.BF16, None, None, None, None, 0, None) == E_NULL
    assert lib.mi_moe_router_fused(None, None, None, 4, 64, 8, 2, _lib.F32, None, None, None, None, 0, None) == E_NULL
    assert lib.mi_moe_router_fused(None, None, None, 4, 64, 300, 2, _lib.BF16, None, None, None, None, 0, None) == E_UNSUP
    assert lib.mi_moe_router_fused(None, None, None, 4, 60, 8, 2, _lib.F32, None, None, None, None, 0, None) == E_UNSUP
    assert lib.mi_moe_router_fused(None, None, None, 4, 72, 8, 2, _lib.BF16, None, None, None, None, 0, None) == E_UNSUP
    assert lib.mi_moe_router_fused(None, None, None, 4, 64, 8, 2, 7, None, None, None, None, 0, None) == E_DTYPE
    assert lib.mi_moe_router_dlogits(None, None, None, None, 4, 8, 9, _lib.BF16, None, None) == E_SHAPE
    assert lib.mi_moe_router_dlogits(None, None, None, None, 4, 8, 2, 7, None, None) == E_DTYPE
    assert lib.mi_moe_router_dlogits(None, None, None, None, 4, 8, 2, _lib.F32, None, None) == E_NULL
    assert lib.mi_moe_router_dlogits(None, None, None, None, 0, 8, 2, _lib.F32, None, None) == 0
    assert lib.mi_moe_router_fused_workspace_bytes(64, 4096, 64) > 0
    assert lib.mi_moe_router_fused_workspace_bytes(32768, 1536, 40) == 0
    # the few-token forms end at 320 tokens where the gate weights fit in LDS, at 1024 where they do not
    assert lib.mi_moe_router_fused_workspace_bytes(320, 1536, 40) > 0
    assert lib.mi_moe_router_fused_workspace_bytes(321, 1536, 40) == 0
    assert lib.mi_moe_router_fused_workspace_bytes(1024, 4096, 64) > 0
    assert lib.mi_moe_router_fused_workspace_bytes(1025, 4096, 64) == 0
    # more than 64 experts: few tokens (the contraction in ranges: groups x ranges x expert blocks x 1 KiB of
    # partial sums, up to 511 groups of 16 tokens), many tokens (T x E >= 2^20: T x E 16-bit logits + 256 bytes),
    # nothing where neither applies; an empty batch needs none
    assert lib.mi_moe_router_fused_workspace_bytes(64, 4096, 128) == 4 * 32 * 8 * 1024
    assert lib.mi_moe_router_fused_workspace_bytes(32768, 2048, 128) == 32768 * 128 * 2 + 256
    assert lib.mi_moe_router_fused_workspace_bytes(8192, 2048, 65) == 0
    assert lib.mi_moe_router_fused_workspace_bytes(0, 4096, 128) == 0
    assert lib.mi_moe_router_fused_sort_workspace_bytes(64, 4096, 64, 6) == lib.mi_moe_router_fused_workspace_bytes(64, 4096, 64) + 256
    assert lib.mi_moe_router_fused_sort_workspace_bytes(2048, 4096, 64, 8) == 0   # many tokens, gate weights beyond LDS
    assert lib.mi_moe_router_fused_sort_workspace_bytes(1024, 1024, 64, 9) == 0   # T * k beyond the one-block sort
    assert lib.mi_moe_router_fused_sort(None, None, None, 2048, 4096, 64, 8, _lib.BF16, None, None, None, None, None,
                                        None, None, 0, None) == E_UNSUP
    assert lib.mi_moe_router_fused_sort(None, None, None, 64, 4096, 64, 6, _lib.BF16, None, None, None, None, None,
                                        None, None, 0, None) == E_NULL
    assert lib.mi_moe_count(None, -1, 8, None, None) == E_SHAPE
    assert lib.mi_moe_sort_bin(None, 4, 2, 0, None, None, None, None, 0, None) == E_SHAPE
    assert lib.mi_moe_sort_bin(None, 4, 2, 8, None, None, None, None, 0, None) == E_NULL
    assert lib.mi_moe_sort_bin_workspace_bytes(1000, 8) == 0  # small inputs need no workspace
    assert lib.mi_moe_sort_bin_workspace_bytes(262144, 40) == (40 * 128 + 40) * 4
    # the non-allocating variant: same checks, and inputs beyond its fixed scratch array are refused on the host
    assert lib.mi_moe_sort_bin_static(None, 4, 2, 0, None, None, None, None) == E_SHAPE
    assert lib.mi_moe_sort_bin_static(None, 4, 2, 8, None, None, None, None) == E_NULL
    assert lib.mi_moe_sort_bin_workspace_bytes(1 << 23, 1000) > (1 << 20)
    assert lib.mi_moe_sort_bin_static(ctypes.c_void_p(256), 1 << 20, 8, 1000, ctypes.c_void_p(256), ctypes.c_void_p(256),
                                      ctypes.c_void_p(256), None) == -7
    assert lib.mi_moe_swiglu_forward(None, None, 4, 12, _lib.BF16, None) == E_UNSUP
    assert lib.mi_moe_swiglu_forward(None, None, 4, 16, 7, None) == E_DTYPE
    assert lib.mi_moe_swiglu_forward(None, None, 4, 6, _lib.F32, None) == E_UNSUP   # fp32 rows: whole 16-byte chunks too
    assert lib.mi_moe_swiglu_forward(None, None, 4, 12, _lib.F32, None) == E_NULL
    # the diagnostic loop probes validate like everything else
    assert lib.mi_moe_probe_kloop(4, None, 4 << 20, 10, None, 0, None) == E_SHAPE
    assert lib.mi_moe_probe_kloop(0, None, 1 << 20, 10, None, 0, None) == E_SHAPE
    assert lib.mi_moe_probe_kloop(0, None, 4 << 20, 10, None, 0, None) == E_NULL
    assert lib.mi_moe_swiglu_forward(None, None, 4, 16, _lib.BF16, None) == E_NULL
    assert lib.mi_moe_swiglu_forward(None, None, 0, 16, _lib.BF16, None) == 0
    assert lib.mi_moe_grouped_wgrad_f32(None, None, None, None, None, None, 16, 8, 8, 0, None) == E_SHAPE
    assert lib.mi_moe_grouped_wgrad_f32(None, None, None, None, None, None, 16, 6, 8, 4, None) == E_UNSUP
    assert lib.mi_moe_grouped_wgrad_f32(None, None, None, None, None, None, 16, 8, 8, 4, None) == E_NULL
    assert lib.mi_moe_grouped_wgrad_naive(None, None, None, None, None, None, 16, 8, 8, 4, 7, None) == E_DTYPE
    assert lib.mi_moe_grouped_wgrad_naive(None, None, None, None, None, None, 16, 8, 8, 4, _lib.F32, None) == E_NULL
    # 16-bit problems the matrix-core kernels cannot take are refused, not run on the slow kernel behind the
    # caller's back: odd K, misaligned pointer
    p16 = ctypes.c_void_p(4096)
    assert lib.mi_moe_scattered_gemm(p16, p16, p16, p16, p16, 16, 12, 8, 4, 2, 0, 1, _lib.BF16, None) == E_UNSUP
    assert lib.mi_moe_scattered_gemm(ctypes.c_void_p(4098), p16, p16, p16, p16, 16, 16, 8, 4, 2, 0, 1, _lib.BF16, None) == -4
    assert lib.mi_moe_scattered_gemm(None, None, None, None, None, 16, 0, 8, 4, 2, 0, 1, _lib.BF16, None) == E_SHAPE
    # the workspace variants: a workspace that is too small (any size is, where no GPU tells the CU count) or
    # misplaced is refused; no workspace is the call without one
    need = lib.mi_moe_grouped_gemm_workspace_bytes()
    assert need == 0 or need % (256 * 256 * 4) == 0
    assert lib.mi_moe_scattered_gemm_ws(p16, p16, p16, p16, p16, 16, 16, 8, 4, 2, 0, 1, _lib.BF16, -1, p16, 8, None) == E_WS
    assert lib.mi_moe_up_swiglu_ws(p16, p16, p16, p16, p16, 16, 16, 8, 4, 2, _lib.BF16, -1, p16, 8, None) == E_WS
    assert lib.mi_moe_scattered_gemm_wt_ws(p16, p16, p16, p16, p16, 16, 16, 8, 4, 2, 0, 1, _lib.BF16, p16, 8, None) == E_WS
    assert lib.mi_moe_scattered_gemm_ws(p16, p16, p16, p16, p16, 16, 12, 8, 4, 2, 0, 1, _lib.BF16, -1, None, 0, None) == E_UNSUP
    assert lib.mi_moe_scattered_gemm(None, None, None, None, None, 16, 8, 8, 4, 2, 0, 1, 7, None) == E_DTYPE
    assert lib.mi_moe_scattered_gemm(None, None, None, None, None, 16, 8, 8, 4, 2, 0, 1, _lib.BF16, None) == E_NULL
    assert lib.mi_moe_scattered_gemm(None, None, None, None, None, 0, 8, 8, 4, 2, 0, 1, _lib.BF16, None) == 0
    assert lib.mi_moe_up_swiglu(None, None, None, None, None, 16, 8, 8, 4, 2, _lib.F16, None) == E_NULL
    assert lib.mi_moe_combine(None, None, None, 4, 0, 8, _lib.BF16, None) == E_SHAPE
    assert lib.mi_moe_combine(None, None, None, 4, 2, 8, 9, None) == E_NULL  # pointers are checked before the dtype
    assert lib.mi_moe_up_swiglu_fp8(None, None, None, None, None, None, 16, 64, 32, 4, 2, _lib.F32, 0, None) == E_DTYPE
    assert lib.mi_moe_down_fp8(None, None, None, None, None, None, 16, 64, 32, 4, _lib.BF16, 0, None) == E_NULL
    assert lib.mi_moe_fp8_tiled_bytes(64, 1408, 4096, 1) == 64 * 2816 * 4096
    assert lib.mi_moe_fp8_tiled_bytes(64, 4096, 1408, 0) == 64 * 4096 * 1408
    assert lib.mi_moe_fp8_tiled_bytes(4, 20, 256, 1) == 4 * 2 * 2 * 4096  # 20 channels pad to two units
    assert lib.mi_moe_fp8_tiled_bytes(4, 20, 200, 1) == 0
    # the same calls with the kernel family chosen by the caller, and the widening pass
    assert lib.mi_moe_up_swiglu_fp8_cfg(None, None, None, None, None, None, 16, 64, 32, 4, 2, _lib.BF16, 0, 2, None) == E_UNSUP
    assert lib.mi_moe_up_swiglu_fp8_cfg(None, None, None, None, None, None, 16, 64, 32, 4, 2, _lib.BF16, 0, 1, None) == E_NULL
    assert lib.mi_moe_down_fp8_cfg(None, None, None, None, None, None, 16, 64, 32, 4, _lib.BF16, 0, -2, None) == E_UNSUP
    assert lib.mi_moe_down_fp8_cfg(None, None, None, None, None, None, 0, 64, 32, 4, _lib.BF16, 0, 1, None) == 0
    assert lib.mi_moe_fp8_dequant(None, None, None, 4, 32, 64, 1, 0, _lib.F32, None) == E_DTYPE
    assert lib.mi_moe_fp8_dequant(None, None, None, 4, 32, 72, 1, 0, _lib.BF16, None) == E_UNSUP   # in % 16
    assert lib.mi_moe_fp8_dequant(None, None, None, 4, 32, 64, 1, 1, _lib.BF16, None) == E_UNSUP   # tiled: in % 128
    assert lib.mi_moe_fp8_dequant(None, None, None, 4, 32, 128, 1, 1, _lib.BF16, None) == E_NULL
    assert lib.mi_moe_fp8_dequant(None, None, None, 0, 32, 128, 1, 1, _lib.BF16, None) == E_SHAPE
    # backward entry points
    assert lib.mi_moe_scattered_gemm_wt(None, None, None, None, None, 16, 128, 8, 4, 2, 0, 1, _lib.F32, None) == E_NULL
    assert lib.mi_moe_scattered_gemm_wt(None, None, None, None, None, 0, 128, 8, 4, 2, 0, 1, _lib.BF16, None) == 0
    assert lib.mi_moe_grouped_wgrad(None, None, None, None, None, None, None, 0, 16, 16, 16, 12, 8, 4, _lib.BF16, None) == E_UNSUP
    assert lib.mi_moe_grouped_wgrad(None, None, None, None, None, None, None, 0, 16, 16, 16, 8, 8, 300, _lib.BF16, None) == E_UNSUP
    assert lib.mi_moe_grouped_wgrad(None, None, None, None, None, None, None, 0, 16, 16, 16, 8, 8, 4, _lib.F32, None) == E_DTYPE
    assert lib.mi_moe_grouped_wgrad(None, None, None, None, None, None, None, 0, 16, 16, 16, 8, 8, 4, _lib.BF16, None) == E_NULL
    assert lib.mi_moe_grouped_wgrad_workspace_bytes(262144, 40, 1024, 1536) > 0
    assert lib.mi_moe_swiglu_backward(None, None, None, None, None, None, None, 4, 12, _lib.BF16, None) == E_UNSUP
    assert lib.mi_moe_swiglu_backward(None, None, None, None, None, None, None, 4, 16, 7, None) == E_DTYPE
    assert lib.mi_moe_swiglu_backward(None, None, None, None, None, None, None, 0, 16, _lib.BF16, None) == 0
    assert lib.mi_moe_combine_grad_gates(None, None, None, 4, 2, 16, _lib.BF16, None) == E_NULL
    assert lib.mi_moe_aux_loss(None, None, None, None, 0, 4, 300, 2, _lib.BF16, None) == E_UNSUP
    assert lib.mi_moe_aux_loss(None, None, None, None, 0, 4, 8, 2, _lib.BF16, None) == E_NULL
    assert lib.mi_moe_aux_loss_workspace_bytes(64, 8) == (2 + 1) * 17 * 4
    assert lib.mi_moe_aux_loss_backward(None, None, None, None, 4, 8, _lib.BF16, None) == E_NULL


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(os.path.dirname(_lib.LIB_PATH), "no_such_lib.so"))
    with pytest.raises(pkg.MiMoeError, match="not found"):
        _lib.load()


# ---------------------------------------------------------------------------------------------------
# toggle
# ---------------------------------------------------------------------------------------------------


def test_kernel_enum_matches_reference_names():
    names = {k.name for k in Kernel}
    assert {"scattermoe", "continuous_count_cute", "swiglu_packed_cute", "rmsnorm_cute", "flash_attention_2",
            "mamba2_ssm", "ladder_residual_overlapped_layer"} <= names
    assert len(names) == 16 and Kernel.scattermoe.value == "scattermoe"


def test_enable_kernels_replaces_and_restores():
    assert not is_kernel_allowed(Kernel.scattermoe)
    with enable_kernels([Kernel.scattermoe]):
        assert is_kernel_allowed(Kernel.scattermoe)
        with enable_kernels({Kernel.rmsnorm_cute}):  # inner context replaces, it does not merge
            assert not is_kernel_allowed(Kernel.scattermoe)
            assert is_kernel_allowed(Kernel.rmsnorm_cute)
        assert is_kernel_allowed(Kernel.scattermoe)
    assert not is_kernel_allowed(Kernel.scattermoe)
    with pytest.raises(ValueError):
        with enable_kernels([Kernel.scattermoe]):
            raise ValueError("boom")
    assert not is_kernel_allowed(Kernel.scattermoe)  # restored even when the block raises


def test_enable_all_cute_kernels_environment_switch(monkeypatch):
    """lm_engine/kernels.py:14-19, 75-76: ENABLE_ALL_CUTE_KERNELS, read when the module is imported, switches every
    kernel on for the whole process -- but only where the kernels can run."""
    from dolomite_engine_amd import kernels

    everything = {k for k in Kernel if k != Kernel.ladder_residual_overlapped_layer}
    before = kernels._KERNELS
    started_with = os.environ.get("ENABLE_ALL_CUTE_KERNELS", "0").lower() in ("1", "true")
    really_available = kernels._kernels_available()
    try:
        for value, available, expect in [(None, True, False), ("0", True, False), ("false", True, False),
                                         ("1", False, False), ("1", True, True), ("TRUE", True, True)]:
            kernels._KERNELS = set()
            if value is None:
                monkeypatch.delenv("ENABLE_ALL_CUTE_KERNELS", raising=False)
            else:
                monkeypatch.setenv("ENABLE_ALL_CUTE_KERNELS", value)
            monkeypatch.setattr(kernels, "_kernels_available", lambda available=available: available)
            assert kernels._enable_all_from_environment() is expect
            assert kernels._KERNELS == (everything if expect else set())
            assert is_kernel_allowed(Kernel.scattermoe) is expect
            assert not is_kernel_allowed(Kernel.ladder_residual_overlapped_layer)
            if expect:  # a context still replaces the set and puts "everything" back
                with enable_kernels([Kernel.rmsnorm_cute]):
                    assert not is_kernel_allowed(Kernel.scattermoe)
                assert is_kernel_allowed(Kernel.scattermoe)
        monkeypatch.setenv("ENABLE_ALL_CUTE_KERNELS", "maybe")
        with pytest.raises(ValueError):
            kernels._enable_all_from_environment()
    finally:
        kernels._KERNELS = before
    # this process was started without the variable (or without a GPU): nothing is on by default
    assert kernels._ENABLE_ALL_KERNELS is (started_with and really_available)


# ---------------------------------------------------------------------------------------------------
# module interface
# ---------------------------------------------------------------------------------------------------


def test_constructor_state_dict_and_init():
    torch.manual_seed(0)
    m = _moe(hidden_size=64, intermediate_size=96, num_experts=8, num_layers=4, initializer_range=0.02)
    sd = m.state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == {
        "gate.weight": (8, 64), "c_fc.weight": (8, 192, 64), "c_proj.weight": (8, 64, 96)}
    assert abs(m.c_fc.weight.std().item() - 0.02) < 2e-3
    assert abs(m.c_proj.weight.std().item() - 0.02 / math.sqrt(2 * 4)) < 1e-3  # std / sqrt(2 * num_layers)
    assert m.top_k == 2 and m.num_experts == 8 and isinstance(m.c_fc, ParameterizedExperts)
    assert m.gate.weight._has_mup_learning_rate and m.c_fc.weight._has_mup_learning_rate
    # non-GLU activation: c_fc has I rows; shared experts add two dense layers; mup scales the std
    m2 = _moe(activation_function="gelu_pytorch_tanh", shared_intermediate_size=40, init_method="mup", m_width=4.0)
    assert m2.c_fc.weight.shape == (8, 48, 32)
    assert m2.c_fc_shared.weight.shape == (40, 32) and m2.c_proj_shared.weight.shape == (32, 40)
    with pytest.raises(ValueError):
        _moe(init_method="bogus")


def test_num_active_parameters():
    m = _moe(hidden_size=32, intermediate_size=48, num_experts=8, num_experts_per_tok=2)
    total = sum(p.numel() for p in m.parameters())
    experts = m.c_fc.weight.numel() + m.c_proj.weight.numel()
    assert m.get_num_active_parameters() == total - experts + experts * 2 // 8


def test_eager_branch_equals_oracle_and_handles_3d_input():
    torch.manual_seed(1)
    m = _moe(hidden_size=32, intermediate_size=48, num_experts=8, num_experts_per_tok=3).eval()
    x = torch.randn(2, 9, 32)
    pkg.clear_aux_loss()
    with torch.no_grad():
        y = m(x)
    assert y.shape == x.shape and pkg.get_aux_loss() == 0 and pkg.is_aux_loss_zero(pkg.get_aux_loss())
    ref = oracle.moe_forward(x.view(-1, 32), m.gate.weight.data, m.c_fc.weight.data, m.c_proj.weight.data, 3)
    torch.testing.assert_close(y.view(-1, 32), ref.y, rtol=1e-5, atol=1e-6)


def test_tiny_config_full_size_eager_equals_oracle():
    """The CPU-runnable benchmark configuration (512 tokens, hidden 256, 8 experts, top-2, intermediate 512, fp32) on the CPU."""
    w = oracle.WORKLOADS["tiny-fp32"]
    inp = oracle.make_inputs(w)
    m = _moe(hidden_size=w.H, intermediate_size=w.I, num_experts=w.E, num_experts_per_tok=w.k,
             use_padding_free_transformer=True).eval()
    with torch.no_grad():
        m.gate.weight.copy_(inp["gate_w"]); m.c_fc.weight.copy_(inp["w_fc"]); m.c_proj.weight.copy_(inp["w_proj"])
        y = m(inp["x"])
    ref = oracle.moe_forward(inp["x"], inp["gate_w"], inp["w_fc"], inp["w_proj"], w.k)
    torch.testing.assert_close(y, ref.y, rtol=1e-4, atol=1e-6)


def test_training_mode_adds_switch_loss():
    torch.manual_seed(2)
    m = _moe().train()
    pkg.clear_aux_loss()
    x = torch.randn(1, 12, 32)
    m(x)
    aux = pkg.get_aux_loss()
    assert isinstance(aux, torch.Tensor) and not pkg.is_aux_loss_zero(aux)
    logits = m.gate(x.view(-1, 32))
    sel = logits.topk(2, -1).indices
    torch.testing.assert_close(aux.detach(), oracle.switch_aux_loss(logits.detach(), sel), rtol=1e-5, atol=1e-6)
    pkg.clear_aux_loss()


def test_router_logit_bias_is_added_before_topk():
    torch.manual_seed(3)
    m = _moe().eval()
    m.router_logit_bias = torch.tensor([9.0, 0, 0, 0, 0, 0, 0, 9.0])
    x = torch.randn(20, 32).view(1, 20, 32)
    with torch.no_grad():
        _, _, sel = m._compute_routing_weights(x.view(-1, 32))
    assert set(sel.flatten().tolist()) == {0, 7}
    assert "router_logit_bias" not in m.state_dict()  # not part of the checkpoint format


def test_kernel_branch_has_no_cpu_fallback():
    m = _moe().eval()
    x = torch.randn(1, 4, 32)
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        with pytest.raises(ValueError, match="GPU"):
            m(x)


def test_fp8_quantisation_eager_path():
    torch.manual_seed(4)
    m = _moe(hidden_size=64, intermediate_size=32).eval()
    x = torch.randn(1, 10, 64)
    w_fc, w_proj = m.c_fc.weight.data.clone(), m.c_proj.weight.data.clone()
    m.quantize_expert_weights_fp8()
    assert m.c_fc.weight is None and m.c_fc.weight_q.dtype == torch.float8_e4m3fn
    assert m.c_fc.weight_scale.shape == (8, 64) and m.c_proj.weight_scale.shape == (8, 64)
    q_fc, s_fc = oracle.quantize_fp8_per_channel(w_fc)
    q_pj, s_pj = oracle.quantize_fp8_per_channel(w_proj)
    assert torch.equal(m.c_fc.weight_q.view(torch.uint8), q_fc.view(torch.uint8))
    with torch.no_grad():
        y = m(x)
    ref = oracle.moe_forward(x.view(-1, 64), m.gate.weight.data, q_fc, q_pj, 2, w_fc_scale=s_fc, w_proj_scale=s_pj)
    torch.testing.assert_close(y.view(-1, 64), ref.y, rtol=1e-4, atol=1e-6)


def test_activation_registry():
    assert pkg.is_glu("swiglu") and pkg.is_glu("geglu") and not pkg.is_glu("gelu")
    act = pkg.get_activation_function("swiglu")
    h = torch.randn(5, 8)
    torch.testing.assert_close(act(h), h[:, :4] * torch.nn.functional.silu(h[:, 4:]))
    assert isinstance(pkg.get_activation_function(None), torch.nn.Identity)
    with pytest.raises(ValueError):
        pkg.get_activation_function("no_such_act")
