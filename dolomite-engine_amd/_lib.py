"""Loader for libmi_moe.so, the C-ABI library holding the gfx950 kernels (include/mi_moe.h).

The library is built in-tree (``csrc/Makefile`` -> ``libmi_moe.so`` next to this file).  There is
no fallback: if the library is missing or a symbol cannot be bound, every kernel entry raises.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi_moe.so")
CSRC_DIR = os.path.join(_HERE, "csrc")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "mi_moe.h")

ABI_VERSION = 1

# dtype codes of include/mi_moe.h
F32, F16, BF16 = 0, 1, 2

_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); must list every function include/mi_moe.h declares
SIGNATURES: dict[str, tuple] = {
    "mi_moe_abi_version": (_i, []),
    "mi_moe_strerror": (ctypes.c_char_p, [_i]),
    "mi_moe_router_topk_softmax": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "mi_moe_router_fused_workspace_bytes": (_sz, [_i, _i, _i]),
    "mi_moe_router_fused": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _sz, _vp]),
    "mi_moe_router_dlogits": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "mi_moe_router_fused_sort_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "mi_moe_router_fused_sort": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "mi_moe_rmsnorm_router_fused_supported": (_i, [_i, _i, _i, _i]),
    "mi_moe_rmsnorm_router_fused": (_i, [_vp, _vp, ctypes.c_float, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "mi_moe_count": (_i, [_vp, _i, _i, _vp, _vp]),
    "mi_moe_sort_bin_workspace_bytes": (_sz, [_i, _i]),
    "mi_moe_sort_bin": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _sz, _vp]),
    "mi_moe_sort_bin_static": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "mi_moe_scattered_gemm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_scattered_gemm_wt": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_scattered_gemm_cfg": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_up_swiglu": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_up_swiglu_cfg": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_grouped_gemm_workspace_bytes": (_sz, []),
    "mi_moe_grouped_gemm_splits": (_i, [_i, _i]),
    "mi_moe_scattered_gemm_ws": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "mi_moe_scattered_gemm_wt_ws": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "mi_moe_up_swiglu_ws": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "mi_moe_up_swiglu_keep": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_combine": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mi_moe_combine_block_tail": (_i, [_vp, _vp, _vp, _vp, ctypes.c_float, _i, _vp, _i, _i, _i, _i, _vp]),
    "mi_moe_swiglu_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "mi_moe_swiglu_forward": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "mi_moe_combine_grad_gates": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mi_moe_grouped_wgrad_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "mi_moe_grouped_wgrad": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_grouped_wgrad_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "mi_moe_grouped_wgrad_naive": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_aux_loss_workspace_bytes": (_sz, [_i, _i]),
    "mi_moe_aux_loss": (_i, [_vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "mi_moe_aux_loss_backward": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "mi_moe_probe_sink_bytes": (_sz, []),
    "mi_moe_probe_kloop": (_i, [_i, _vp, _sz, _i, _vp, _sz, _vp]),
    "mi_moe_fp8_tiled_bytes": (_sz, [_i, _i, _i, _i]),
    "mi_moe_up_swiglu_fp8": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_down_fp8": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_fp8_dequant": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_up_swiglu_fp8_cfg": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "mi_moe_down_fp8_cfg": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
}

# return codes of include/mi_moe.h that callers branch on
MI_MOE_EDTYPE = -3
MI_MOE_EALIGN = -4
MI_MOE_EUNSUPPORTED = -6
MI_MOE_ETOOLARGE = -7

_lib = None
_lock = threading.Lock()


class MiMoeError(RuntimeError):
    """A C-ABI call returned a non-zero code."""


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 into libmi_moe.so (always recompiles)."""
    jobs = str(min(8, os.cpu_count() or 1))
    subprocess.run(["make", "-C", CSRC_DIR, "clean"], check=True, capture_output=not verbose)
    proc = subprocess.run(["make", "-C", CSRC_DIR, "-j", jobs], capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode != 0 or not os.path.exists(LIB_PATH):
        raise RuntimeError("building libmi_moe.so failed")
    global _lib
    _lib = None
    return LIB_PATH


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def load() -> ctypes.CDLL:
    """Return the bound library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise MiMoeError(
                f"{LIB_PATH} not found: build it with `make -C {CSRC_DIR}` "
                "(the scattermoe kernel path has no fallback)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError names the missing symbol
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.mi_moe_abi_version()
        if got != ABI_VERSION:
            raise MiMoeError(f"libmi_moe.so has ABI version {got}, this package expects {ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise MiMoeError(load().mi_moe_strerror(rc).decode())
