"""Tensor-level wrappers over the C ABI (include/mi_moe.h).

``scattered_experts`` and ``continuous_count`` keep the call signatures the reference uses for the
external ops it imports at lm_engine/hf_models/modeling_utils/mlp_blocks/moe.py:22-24 (call sites
moe.py:40 and moe.py:91-101), so either can be bound in their place.  The remaining functions are
the fused stages the MoE module of this package calls.

PyTorch is used for device memory and the current stream only; every function enqueues HIP
kernels on ``torch.cuda.current_stream()`` and returns without synchronising.  None of these functions
records a gradient: tensors that require grad are refused while grad mode is on (the differentiable
compositions are in ``autograd.py``).
"""

from __future__ import annotations

import torch

from . import _lib
from ._lib import BF16, F16, F32, check

_DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}


_TIMER = None
_WARNED: set = set()


def _warn_once(key, message: str) -> None:
    """Slow paths are taken loudly: one warning per process and key (reason, shape, dtype)."""
    if key not in _WARNED:
        _WARNED.add(key)
        import warnings

        warnings.warn(message, RuntimeWarning, stacklevel=3)


def set_stage_timer(timer) -> None:
    """Install an object with ``begin(name)`` / ``end(name)`` that is called around every kernel
    stage (used by the benchmark to put HIP events on the launch stream); ``None`` removes it."""
    global _TIMER
    _TIMER = timer


class _stage:
    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        if _TIMER is not None:
            _TIMER.begin(self.name)

    def __exit__(self, *exc):
        if _TIMER is not None:
            _TIMER.end(self.name)
        return False


def is_available() -> bool:
    """True when a GPU is visible and the kernel library has been built."""
    return torch.cuda.is_available() and _lib.is_built()


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype} (float32, float16 and bfloat16 are supported)") from None


# torch.cuda.current_stream() / current_device() walk several Python layers (8 us per call, four calls per layer
# forward); the C entry points underneath them return the same handle / index in a fraction of a microsecond.
_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_RAW_DEVICE = getattr(torch._C, "_cuda_getDevice", None)


def _current_device() -> int:
    return _RAW_DEVICE() if _RAW_DEVICE is not None else torch.cuda.current_device()


def _stream() -> int:
    if _RAW_STREAM is not None:
        return _RAW_STREAM(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(*tensors: torch.Tensor | None) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("the scattermoe kernels need tensors on the GPU (no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError("all tensors must be on the same device")
    if dev is not None and dev.index is not None and dev.index != _current_device():
        raise ValueError("tensors must be on the current device")


def _no_grad(*tensors: torch.Tensor | None) -> None:
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        raise RuntimeError(
            "the MI355X scattermoe kernels are forward-only (they record no gradient): run under torch.no_grad() / "
            "inference_mode(), or go through the module / autograd.py"
        )


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _i32(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.int32 else t.to(torch.int32)


def _native_weight(expert_weights: torch.Tensor) -> torch.Tensor:
    """(E, in, out) view as passed by the reference -> contiguous (E, out, in) storage, without a copy
    when the argument is the permuted view of the module's parameter."""
    w = expert_weights.permute(0, 2, 1)
    return w if w.is_contiguous() else w.contiguous()


# ------------------------------------------------------------------------------------------------
# routing
# ------------------------------------------------------------------------------------------------


def router_topk_softmax(logits: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Top-k (value descending, expert index ascending) + fp32 softmax over the k values.

    logits (T, E) -> gates (T, k) in logits.dtype, experts (T, k) int32."""
    _dev(logits)
    _no_grad(logits)
    logits = logits.contiguous()
    T, E = logits.shape
    gates = torch.empty((T, k), dtype=logits.dtype, device=logits.device)
    idx = torch.empty((T, k), dtype=torch.int32, device=logits.device)
    with _stage("router_topk_softmax"):
        check(_lib.load().mi_moe_router_topk_softmax(_ptr(logits), T, E, k, _code(logits.dtype), _ptr(gates), _ptr(idx),
                                                    _stream()))
    return gates, idx


def _router_streaming_supported(x: torch.Tensor, num_experts: int, k: int) -> bool:
    """The streaming kernels of the fused router (gate weights in LDS, the split-K small-batch form, the forms with
    the sort or the RMSNorm folded in): 16-bit, at most 64 experts, k <= 8."""
    return (x.dtype in (torch.bfloat16, torch.float16) and num_experts <= 64 and k <= 8 and x.shape[-1] % 16 == 0)


def router_fused_supported(x: torch.Tensor, num_experts: int, k: int) -> bool:
    """What :func:`router_fused` takes: the streaming kernels' shapes, and through the general kernel fp32
    (H % 8 == 0), up to 256 experts and k up to 64 (16-bit: H % 16 == 0)."""
    if _router_streaming_supported(x, num_experts, k):
        return True
    if not (1 <= k <= min(num_experts, 64) and num_experts <= 256):
        return False
    if x.dtype == torch.float32:
        return x.shape[-1] % 8 == 0
    return x.dtype in (torch.bfloat16, torch.float16) and x.shape[-1] % 16 == 0


def router_fused(x: torch.Tensor, gate_weight: torch.Tensor, k: int, bias: torch.Tensor | None = None,
                 return_logits: bool = False, split_k: bool = True):
    """logits = x @ gate_weight^T (+bias) in x.dtype, top-k, softmax: one pass over x.

    ``split_k=False`` withholds the workspace, i.e. forces the single-launch kernel for few tokens too.
    Returns (logits or None, gates (T,k), experts (T,k) int32)."""
    _dev(x, gate_weight, bias)
    _no_grad(x, gate_weight)
    x = x.contiguous()
    gate_weight = gate_weight.contiguous()
    T, H = x.shape
    E = gate_weight.shape[0]
    if gate_weight.dtype != x.dtype or gate_weight.shape[1] != H:
        raise ValueError("gate weight must be (E, H) in the dtype of x")
    if bias is not None:
        bias = bias.to(torch.float32).contiguous()
    logits = torch.empty((T, E), dtype=x.dtype, device=x.device) if return_logits else None
    gates = torch.empty((T, k), dtype=x.dtype, device=x.device)
    idx = torch.empty((T, k), dtype=torch.int32, device=x.device)
    lib = _lib.load()
    # non-zero for few tokens (K split over the chip) and, with more than 64 experts, for many tokens (16-bit: the
    # logits come from the grouped GEMM's tile kernels, then the top-k kernel)
    ws_bytes = lib.mi_moe_router_fused_workspace_bytes(T, H, E) if (
        split_k and (_router_streaming_supported(x, E, k) or E > 64)) else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    with _stage("router_fused"):
        check(lib.mi_moe_router_fused(_ptr(x), _ptr(gate_weight), _ptr(bias), T, H, E, k, _code(x.dtype),
                                     _ptr(logits), _ptr(gates), _ptr(idx), _ptr(ws), ws_bytes, _stream()))
    return logits, gates, idx


def router_fused_sort_supported(x: torch.Tensor, num_experts: int, k: int) -> bool:
    """Whether :func:`router_fused_sort` takes the shape: few tokens (split-K router whose finishing launch sorts,
    T <= 320, or T <= 1024 with T * k <= 8192 where the gate weights do not fit in LDS), or gate weights that fit
    in LDS (the router counts the experts for the sort's two remaining passes)."""
    if not (_router_streaming_supported(x, num_experts, k) and x.is_cuda and x.dim() == 2 and x.shape[0] >= 1):
        return False
    return _lib.load().mi_moe_router_fused_sort_workspace_bytes(x.shape[0], x.shape[1], num_experts, k) > 0


def router_fused_sort(x: torch.Tensor, gate_weight: torch.Tensor, k: int, bias: torch.Tensor | None = None,
                      return_logits: bool = False):
    """:func:`router_fused` and :func:`sort_bin` in two launches instead of three (the router's finishing launch
    sorts as well).  Returns (logits or None, gates (T, k), experts (T, k) int32, sorted_expert_idxs (L,),
    sorted_scattered_idxs (L,), expert_offsets (E,)), identical to the separate calls."""
    _dev(x, gate_weight, bias)
    _no_grad(x, gate_weight)
    x = x.contiguous()
    gate_weight = gate_weight.contiguous()
    T, H = x.shape
    E = gate_weight.shape[0]
    if gate_weight.dtype != x.dtype or gate_weight.shape[1] != H:
        raise ValueError("gate weight must be (E, H) in the dtype of x")
    if bias is not None:
        bias = bias.to(torch.float32).contiguous()
    dev = x.device
    logits = torch.empty((T, E), dtype=x.dtype, device=dev) if return_logits else None
    gates = torch.empty((T, k), dtype=x.dtype, device=dev)
    idx = torch.empty((T, k), dtype=torch.int32, device=dev)
    se = torch.empty(T * k, dtype=torch.int32, device=dev)
    ss = torch.empty(T * k, dtype=torch.int32, device=dev)
    off = torch.empty(E, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.mi_moe_router_fused_sort_workspace_bytes(T, H, E, k)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    with _stage("router_fused_sort"):
        check(lib.mi_moe_router_fused_sort(_ptr(x), _ptr(gate_weight), _ptr(bias), T, H, E, k, _code(x.dtype),
                                          _ptr(logits), _ptr(gates), _ptr(idx), _ptr(se), _ptr(ss), _ptr(off),
                                          _ptr(ws), ws_bytes, _stream()))
    return logits, gates, idx, se, ss, off


def rmsnorm_router_fused_supported(x: torch.Tensor, num_experts: int, k: int) -> bool:
    return (x.dtype in (torch.bfloat16, torch.float16) and x.is_cuda
            and bool(_lib.load().mi_moe_rmsnorm_router_fused_supported(x.shape[-1], num_experts, k, _code(x.dtype))))


def rmsnorm_router_fused(h: torch.Tensor, ln_weight: torch.Tensor | None, eps: float, gate_weight: torch.Tensor,
                         k: int, bias: torch.Tensor | None = None, return_logits: bool = False):
    """RMSNorm (torch.nn.RMSNorm semantics: fp32 arithmetic, one rounding) + fused router in one kernel.

    Stands in for ``ln_2`` followed by the routing of the layer (mixins/dense/layer.py:58-59, moe.py:246-257).
    Returns (x_norm (T, H), logits or None, gates (T, k), experts (T, k) int32)."""
    _dev(h, ln_weight, gate_weight, bias)
    _no_grad(h, gate_weight)
    h = h.contiguous()
    gate_weight = gate_weight.contiguous()
    T, H = h.shape
    E = gate_weight.shape[0]
    if gate_weight.dtype != h.dtype or gate_weight.shape[1] != H:
        raise ValueError("gate weight must be (E, H) in the dtype of h")
    if ln_weight is not None:
        if ln_weight.shape != (H,):
            raise ValueError("ln_weight must be (H,)")
        ln_weight = ln_weight.to(h.dtype).contiguous()
    if bias is not None:
        bias = bias.to(torch.float32).contiguous()
    x_norm = torch.empty_like(h)
    logits = torch.empty((T, E), dtype=h.dtype, device=h.device) if return_logits else None
    gates = torch.empty((T, k), dtype=h.dtype, device=h.device)
    idx = torch.empty((T, k), dtype=torch.int32, device=h.device)
    with _stage("rmsnorm_router_fused"):
        check(_lib.load().mi_moe_rmsnorm_router_fused(_ptr(h), _ptr(ln_weight), float(eps), _ptr(gate_weight), _ptr(bias),
                                                     T, H, E, k, _code(h.dtype), _ptr(x_norm), _ptr(logits),
                                                     _ptr(gates), _ptr(idx), _stream()))
    return x_norm, logits, gates, idx


def router_dlogits(logits: torch.Tensor, experts: torch.Tensor, d_gates: torch.Tensor | None,
                   d_logits_extra: torch.Tensor | None) -> torch.Tensor:
    """Gradient of the router's outputs w.r.t. the (T, E) logits: the softmax over the k picked logits backwards,
    scattered to the picked experts, plus ``d_logits_extra`` (the gradient that reaches the logits directly, i.e.
    the auxiliary loss).  ``experts`` (T, k) int32, ``d_gates`` (T, k) or None, all floating tensors in
    logits.dtype.  The element-wise part of the backward of moe.py:246-257."""
    _dev(logits, experts, d_gates, d_logits_extra)
    _no_grad(logits, d_gates, d_logits_extra)
    logits = logits.contiguous()
    experts = _i32(experts).contiguous()
    T, E = logits.shape
    k = experts.shape[1]
    if experts.shape[0] != T:
        raise ValueError("experts must be (T, k)")
    for name, t, shape in (("d_gates", d_gates, (T, k)), ("d_logits_extra", d_logits_extra, (T, E))):
        if t is not None and (tuple(t.shape) != shape or t.dtype != logits.dtype):
            raise ValueError(f"{name} must be {shape} in the dtype of the logits")
    d_gates = None if d_gates is None else d_gates.contiguous()
    d_logits_extra = None if d_logits_extra is None else d_logits_extra.contiguous()
    out = torch.empty_like(logits)
    with _stage("router_dlogits"):
        check(_lib.load().mi_moe_router_dlogits(_ptr(logits), _ptr(experts), _ptr(d_gates), _ptr(d_logits_extra), T, E, k,
                                               _code(logits.dtype), _ptr(out), _stream()))
    return out


def continuous_count(x: torch.Tensor, size: int) -> torch.Tensor:
    """Histogram of the integer tensor ``x`` with ``size`` bins, uint32 (moe.py:38-44)."""
    _dev(x)
    ids = _i32(x.flatten()).contiguous()
    out = torch.empty(size, dtype=torch.uint32, device=x.device)
    with _stage("count"):
        check(_lib.load().mi_moe_count(_ptr(ids), ids.numel(), size, _ptr(out), _stream()))
    return out


def sort_bin(selected_experts: torch.Tensor, num_experts: int):
    """Stable expert sort + inclusive offsets (moe.py:263-271).

    selected_experts (T, k) integer -> (sorted_expert_idxs (L,), sorted_scattered_idxs (L,),
    expert_offsets (E,)), all int32."""
    _dev(selected_experts)
    T, k = selected_experts.shape
    ids = _i32(selected_experts).contiguous()
    L = T * k
    dev = ids.device
    se = torch.empty(L, dtype=torch.int32, device=dev)
    ss = torch.empty(L, dtype=torch.int32, device=dev)
    off = torch.empty(num_experts, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.mi_moe_sort_bin_workspace_bytes(L, num_experts)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    with _stage("sort_bin"):
        check(lib.mi_moe_sort_bin(_ptr(ids), T, k, num_experts, _ptr(se), _ptr(ss), _ptr(off), _ptr(ws), ws_bytes,
                                  _stream()))
    return se, ss, off


# ------------------------------------------------------------------------------------------------
# experts
# ------------------------------------------------------------------------------------------------


_GEMM_WS: dict = {}
_GEMM_WS_MAX = 16


def _gemm_workspace(device: torch.device, K: int, dtype: torch.dtype, enabled: bool = True):
    """(tensor, bytes) of the workspace that lets the persistent grouped GEMM cut the tiles of its last, partly
    filled round along K (mi_moe_grouped_gemm_workspace_bytes: one fp32 partial tile per CU, 64 MiB on 256 CUs), or
    (None, 0) when the library would not use it for this contraction length and dtype (mi_moe_grouped_gemm_splits:
    16-bit and K >= 5120) -- most layers never allocate one.

    One buffer per (device, stream), created on first use and NEVER released: a HIP graph captured on that stream
    holds the buffer's address for as long as it can be replayed.  After _GEMM_WS_MAX buffers further streams get
    none (their calls run every tile whole, which is only slower)."""
    if not enabled or dtype not in (torch.float16, torch.bfloat16):
        return None, 0
    lib = _lib.load()
    if not lib.mi_moe_grouped_gemm_splits(K, _code(dtype)):
        return None, 0
    key = (device.index, _stream())
    ws = _GEMM_WS.get(key)
    if ws is None:
        n = lib.mi_moe_grouped_gemm_workspace_bytes()
        if n == 0 or len(_GEMM_WS) >= _GEMM_WS_MAX:
            return None, 0
        ws = torch.empty(n, dtype=torch.uint8, device=device)
        _GEMM_WS[key] = ws
    return ws, ws.numel()


def scattered_gemm(inputs: torch.Tensor, weight: torch.Tensor, k: int, sorted_scattered_idxs: torch.Tensor,
                   expert_offsets: torch.Tensor, grouped_in: bool, grouped_out: bool, cfg: int = -1,
                   weight_kn: bool = False, split_k: bool = True) -> torch.Tensor:
    """Grouped GEMM with the weight in native (E, out, in) layout; returns (L, out).

    ``split_k``: hand the persistent kernel its workspace (see _gemm_workspace); False runs every tile whole.

    ``weight_kn``: the weight is (E, in, out) instead (``inputs @ weight[e]``, the form of the backward's data
    gradients).  Shapes the transposed-weight kernel does not take are transposed once and run the normal way."""
    _dev(inputs, weight, sorted_scattered_idxs, expert_offsets)
    _no_grad(inputs, weight)
    inputs = inputs.contiguous()
    weight = weight.contiguous()
    ss = _i32(sorted_scattered_idxs).contiguous()
    off = _i32(expert_offsets).contiguous()
    if weight_kn:
        E, K, N = weight.shape
    else:
        E, N, K = weight.shape
    if inputs.shape[1] != K or weight.dtype != inputs.dtype:
        raise ValueError("inputs must be (rows, in_features) in the dtype of the weights")
    L = ss.numel()
    if grouped_in and inputs.shape[0] != L:
        raise ValueError("grouped inputs must have one row per sorted slot")
    if not grouped_in and inputs.shape[0] * k != L:
        raise ValueError("scattered inputs must have L / k rows")
    out = torch.empty((L, N), dtype=inputs.dtype, device=inputs.device)
    lib = _lib.load()
    ws, ws_bytes = _gemm_workspace(inputs.device, K, inputs.dtype, split_k)
    if weight_kn:
        with _stage("scattered_gemm"):
            rc = lib.mi_moe_scattered_gemm_wt_ws(_ptr(inputs), _ptr(weight), _ptr(out), _ptr(ss), _ptr(off), L, K, N,
                                                 E, k, int(grouped_in), int(grouped_out), _code(inputs.dtype),
                                                 _ptr(ws), ws_bytes, _stream())
        if rc == 0:
            return out
        if rc not in (_lib.MI_MOE_EUNSUPPORTED, _lib.MI_MOE_EDTYPE, _lib.MI_MOE_EALIGN):
            check(rc)
        if inputs.dtype != torch.float32:
            # (fp32 has no transposed-weight kernel: its transposed copy is the regular path, not a refusal)
            _warn_once(("weight_kn", rc, K, N, inputs.dtype),
                       f"scattered_gemm(weight_kn=True): the transposed-weight kernel does not take "
                       f"K={K}, N={N}, E={E}, {inputs.dtype} ({lib.mi_moe_strerror(rc).decode()}); making a "
                       "transposed copy of the weights for this call")
        weight = weight.transpose(1, 2).contiguous()
    with _stage("scattered_gemm"):
        rc = _gemm_or_slow(lambda c: lib.mi_moe_scattered_gemm_ws(
            _ptr(inputs), _ptr(weight), _ptr(out), _ptr(ss), _ptr(off), L, K, N, E, k, int(grouped_in),
            int(grouped_out), _code(inputs.dtype), c, _ptr(ws), ws_bytes, _stream()), cfg, K, N, inputs.dtype,
            inputs.shape[0])
        check(rc)
    return out


def _gemm_or_slow(call, cfg: int, K: int, N: int, dtype: torch.dtype, rows: int) -> int:
    """Run ``call(cfg)``.  The library refuses problems its matrix-core kernels cannot take instead of silently
    running them on the one-thread-per-output kernel; the reference's op takes any shape, so for an automatic pick
    (cfg < 0) a refusal for the shape's granularity (K not a multiple of a 16-byte chunk, N % 4) or for a misaligned
    pointer is answered here by asking for that kernel explicitly -- with a warning per (reason, K, N, dtype) whose
    text is the library's.  A well-formed problem that is refused only because an operand is too large for the
    kernels' 32-bit element offsets is NOT sent there (it would run orders of magnitude slower without a word): it
    raises, and the caller splits the rows."""
    rc = call(cfg)
    if cfg < 0 and rc in (_lib.MI_MOE_EUNSUPPORTED, _lib.MI_MOE_EALIGN):
        chunk = 4 if dtype == torch.float32 else 8
        if rc == _lib.MI_MOE_EUNSUPPORTED and K % chunk == 0 and N % 4 == 0:
            raise _lib.MiMoeError(
                f"grouped GEMM with {rows} input rows, K={K}, N={N}, {dtype}: an operand has 2^31 or more elements, "
                "beyond the 32-bit element offsets of the matrix-core kernels; split the call by rows")
        _warn_once(("slow_gemm", rc, K, N, dtype),
                   f"grouped GEMM with K={K}, N={N}, {dtype}: {_lib.load().mi_moe_strerror(rc).decode()}; running "
                   "the one-thread-per-output kernel instead")
        rc = call(3)
    return rc


def combine(o: torch.Tensor, gates: torch.Tensor, shared: torch.Tensor | None = None,
            residual: torch.Tensor | None = None, residual_scale: float | None = None) -> torch.Tensor:
    """y[t] = sum_j gates[t, j] * o[t*k + j]  with o (T*k, H), gates (T, k).

    Optionally folds the tail of the transformer block into the same pass, each step rounded to the
    dtype like the separate torch operations: ``+ shared`` (shared-expert output, moe.py:214),
    ``* residual_scale`` (m_residual) and ``+ residual`` (mixins/dense/layer.py:61-66)."""
    _dev(o, gates, shared, residual)
    _no_grad(o, gates)
    o = o.contiguous()
    gates = gates.contiguous()
    T, k = gates.shape
    H = o.shape[1]
    if o.shape[0] != T * k or gates.dtype != o.dtype:
        raise ValueError("o must be (T*k, H) and gates (T, k) of the same dtype")
    for name, t in (("shared", shared), ("residual", residual)):
        if t is not None and (tuple(t.shape) != (T, H) or t.dtype != o.dtype):
            raise ValueError(f"{name} must be (T, H) in the dtype of o")
    y = torch.empty((T, H), dtype=o.dtype, device=o.device)
    with _stage("combine"):
        if shared is None and residual is None and residual_scale is None:
            check(_lib.load().mi_moe_combine(_ptr(o), _ptr(gates), _ptr(y), T, k, H, _code(o.dtype), _stream()))
        else:
            shared = None if shared is None else shared.contiguous()
            residual = None if residual is None else residual.contiguous()
            check(_lib.load().mi_moe_combine_block_tail(
                _ptr(o), _ptr(gates), _ptr(shared), _ptr(residual),
                1.0 if residual_scale is None else float(residual_scale), int(residual_scale is not None),
                _ptr(y), T, k, H, _code(o.dtype), _stream()))
    return y


def elementwise_supported(dtype: torch.dtype, row_length: int) -> bool:
    """Shapes the element-wise forward / backward kernels take: rows of whole 16-byte chunks."""
    if dtype == torch.float32:
        return row_length % 4 == 0
    return dtype in (torch.float16, torch.bfloat16) and row_length % 8 == 0


def swiglu_forward(h: torch.Tensor) -> torch.Tensor:
    """``h[:, :I] * silu(h[:, I:])`` for a stored pre-activation h (L, 2I) (activations/glu.py:42-43): fp32
    arithmetic on the rounded h, one rounding.  Rows of whole 16-byte chunks (I % 8 == 0; fp32: I % 4 == 0) run the
    kernel, a ragged I runs torch."""
    _dev(h)
    _no_grad(h)
    h = h.contiguous()
    L, I2 = h.shape
    I = I2 // 2
    if I2 % 2:
        raise ValueError("h must be (L, 2I)")
    if not elementwise_supported(h.dtype, I):
        up, gate = h[:, :I].float(), h[:, I:].float()
        return (up * gate * torch.sigmoid(gate)).to(h.dtype)
    act = torch.empty((L, I), dtype=h.dtype, device=h.device)
    with _stage("swiglu_forward"):
        check(_lib.load().mi_moe_swiglu_forward(_ptr(h), _ptr(act), L, I, _code(h.dtype), _stream()))
    return act


def swiglu_backward(h: torch.Tensor, d_act: torch.Tensor, gates: torch.Tensor | None = None,
                    sorted_scattered_idxs: torch.Tensor | None = None, want_act: bool = False,
                    want_gate_grad: bool = False):
    """Backward of ``a = h[:, :I] * silu(h[:, I:])`` (activations/glu.py:42-43) over the sorted rows.

    ``d_act`` (L, I) is the gradient w.r.t. ``a`` before the router weight; row i is scaled by
    ``g_i = gates.flatten()[sorted_scattered_idxs[i]]`` (1 without ``gates``).  Returns ``(d_h, act_g, d_gates)``:
    ``d_h`` (L, 2I); ``act_g = g * a`` (L, I) if ``want_act``; ``d_gates`` in the shape of ``gates`` with
    ``<d_act[i], a[i]>`` at the slot of row i if ``want_gate_grad``.  Shapes: :func:`elementwise_supported`."""
    _dev(h, d_act, gates, sorted_scattered_idxs)
    _no_grad(h, d_act)
    h = h.contiguous()
    d_act = d_act.contiguous()
    L, I = d_act.shape
    if tuple(h.shape) != (L, 2 * I) or h.dtype != d_act.dtype:
        raise ValueError("h must be (L, 2I) and d_act (L, I) of the same dtype")
    if gates is not None:
        gates = gates.contiguous()
        if gates.numel() != L or gates.dtype != h.dtype:
            raise ValueError("gates must have one entry per row in the dtype of h")
    if sorted_scattered_idxs is not None:
        sorted_scattered_idxs = sorted_scattered_idxs.contiguous()
        if tuple(sorted_scattered_idxs.shape) != (L,) or sorted_scattered_idxs.dtype != torch.int32:
            raise ValueError("sorted_scattered_idxs must be (L,) int32")
    if want_gate_grad and gates is None:
        raise ValueError("want_gate_grad needs gates")
    d_h = torch.empty_like(h)
    act_g = torch.empty_like(d_act) if want_act else None
    d_gates = torch.empty_like(gates) if want_gate_grad else None
    with _stage("swiglu_backward"):
        check(_lib.load().mi_moe_swiglu_backward(_ptr(h), _ptr(d_act), _ptr(gates), _ptr(sorted_scattered_idxs),
                                                 _ptr(d_h), _ptr(act_g), _ptr(d_gates), L, I, _code(h.dtype),
                                                 _stream()))
    return d_h, act_g, d_gates


def combine_grad_gates(o: torch.Tensor, dy: torch.Tensor, k: int) -> torch.Tensor:
    """d_gates[t, j] = <dy[t], o[t*k + j]>: the gradient of :func:`combine` w.r.t. the gates.  Shapes:
    :func:`elementwise_supported`."""
    _dev(o, dy)
    _no_grad(o, dy)
    o = o.contiguous()
    dy = dy.contiguous()
    T, H = dy.shape
    if tuple(o.shape) != (T * k, H) or o.dtype != dy.dtype:
        raise ValueError("o must be (T*k, H) and dy (T, H) of the same dtype")
    d_gates = torch.empty((T, k), dtype=o.dtype, device=o.device)
    with _stage("combine_grad_gates"):
        check(_lib.load().mi_moe_combine_grad_gates(_ptr(o), _ptr(dy), _ptr(d_gates), T, k, H, _code(o.dtype),
                                                    _stream()))
    return d_gates


def grouped_wgrad_supported(a: torch.Tensor, b: torch.Tensor, num_experts: int) -> bool:
    return (a.dtype in (torch.float16, torch.bfloat16) and a.shape[1] % 8 == 0 and b.shape[1] % 8 == 0
            and num_experts <= 256 and a.numel() * 2 < 2 ** 32 and b.numel() * 2 < 2 ** 32)


def grouped_wgrad(a: torch.Tensor, b: torch.Tensor, expert_offsets: torch.Tensor,
                  a_idx: torch.Tensor | None = None, b_idx: torch.Tensor | None = None) -> torch.Tensor:
    """dw[e] = sum over the sorted rows r of expert e of outer(a[ai(r)], b[bi(r)]), (E, M, N).

    ``a`` (rows_a, M) and ``b`` (rows_b, N); ``a_idx`` / ``b_idx`` (L,) int32 map a sorted row to a row of the
    operand (``None``: the operand is already in sorted order and has L rows).  The per-expert weight gradient of
    the backward of ``scattered_experts`` (moe.py:91-101).  16-bit operands with M % 8 == N % 8 == 0 and fp32 operands
    with M % 4 == N % 4 == 0 run on the matrix cores; other shapes on a one-thread-per-element kernel."""
    _dev(a, b, expert_offsets, a_idx, b_idx)
    _no_grad(a, b)
    a = a.contiguous()
    b = b.contiguous()
    E = expert_offsets.shape[0]
    M, N = a.shape[1], b.shape[1]
    if a.dtype != b.dtype:
        raise ValueError("a and b must have the same dtype")
    L = None
    for t, i in ((a, a_idx), (b, b_idx)):
        n = t.shape[0] if i is None else i.shape[0]
        if i is not None and (i.dtype != torch.int32 or i.dim() != 1):
            raise ValueError("index arrays must be 1-D int32")
        if L is not None and n != L:
            raise ValueError("a and b disagree on the number of sorted rows")
        L = n
    a_idx = None if a_idx is None else a_idx.contiguous()
    b_idx = None if b_idx is None else b_idx.contiguous()
    expert_offsets = _i32(expert_offsets).contiguous()
    lib = _lib.load()
    if a.dtype == torch.float32 and M % 4 == 0 and N % 4 == 0 and E <= 65535:
        # fp32 on its own matrix instruction: one workgroup per (expert, tile) adds the rows in order, no workspace
        dw = torch.empty((E, M, N), dtype=a.dtype, device=a.device)
        with _stage("grouped_wgrad"):
            check(lib.mi_moe_grouped_wgrad_f32(_ptr(a), _ptr(a_idx), _ptr(b), _ptr(b_idx), _ptr(expert_offsets), _ptr(dw),
                                               L, M, N, E, _stream()))
        return dw
    if not grouped_wgrad_supported(a, b, E):
        # odd shapes: the one-thread-per-element kernel, on the device like everything else (no per-expert host
        # loop, no synchronisation)
        if a.dtype != torch.float32:
            _warn_once("slow_wgrad", f"grouped weight gradient with M={M}, N={N}, E={E}, {a.dtype}: running the slow "
                       "one-thread-per-element kernel (the matrix-core kernel needs M % 8 == N % 8 == 0, E <= 256)")
        dw = torch.empty((E, M, N), dtype=a.dtype, device=a.device)
        with _stage("grouped_wgrad"):
            check(lib.mi_moe_grouped_wgrad_naive(_ptr(a), _ptr(a_idx), _ptr(b), _ptr(b_idx), _ptr(expert_offsets),
                                                 _ptr(dw), L, M, N, E, _code(a.dtype), _stream()))
        return dw
    ws_bytes = int(lib.mi_moe_grouped_wgrad_workspace_bytes(L, E, M, N))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=a.device)
    dw = torch.empty((E, M, N), dtype=a.dtype, device=a.device)
    with _stage("grouped_wgrad"):
        check(lib.mi_moe_grouped_wgrad(_ptr(a), _ptr(a_idx), _ptr(b), _ptr(b_idx), _ptr(expert_offsets), _ptr(dw),
                                       _ptr(ws), ws_bytes, L, a.shape[0], b.shape[0], M, N, E, _code(a.dtype),
                                       _stream()))
    return dw


def aux_loss_supported(logits: torch.Tensor) -> bool:
    return logits.is_cuda and logits.dim() == 2 and logits.shape[0] >= 1 and 1 <= logits.shape[1] <= 256 and \
        logits.dtype in (torch.float32, torch.float16, torch.bfloat16)


def aux_loss(logits: torch.Tensor, topk_idxs: torch.Tensor) -> torch.Tensor:
    """Switch + z auxiliary loss of moe.py:346-369 (single data-parallel rank) from the (T, E) logits and the
    (T, k) selected experts.  Returns 1 + E floats: [0] the loss, [1:] d loss / d (summed probabilities), which
    :func:`aux_loss_backward` takes."""
    _dev(logits, topk_idxs)
    _no_grad(logits)
    logits = logits.contiguous()
    idx = _i32(topk_idxs).contiguous()
    T, E = logits.shape
    if idx.dim() != 2 or idx.shape[0] != T:
        raise ValueError("topk_idxs must be (T, k)")
    lib = _lib.load()
    ws_bytes = int(lib.mi_moe_aux_loss_workspace_bytes(T, E))
    ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=logits.device)
    loss_w = torch.empty(1 + E, dtype=torch.float32, device=logits.device)
    with _stage("aux_loss"):
        check(lib.mi_moe_aux_loss(_ptr(logits), _ptr(idx), _ptr(loss_w), _ptr(ws), ws_bytes, T, E, idx.shape[1],
                                  _code(logits.dtype), _stream()))
    return loss_w


def aux_loss_backward(logits: torch.Tensor, loss_w: torch.Tensor, grad: torch.Tensor) -> torch.Tensor:
    """Gradient of :func:`aux_loss` w.r.t. the logits, scaled by the scalar ``grad``."""
    _dev(logits, loss_w, grad)
    _no_grad(logits)
    logits = logits.contiguous()
    T, E = logits.shape
    if loss_w.dtype != torch.float32 or loss_w.numel() != 1 + E:
        raise ValueError("loss_w must be the 1 + E floats aux_loss returned")
    grad = grad.detach().to(torch.float32).reshape(1).contiguous()
    d_logits = torch.empty_like(logits)
    with _stage("aux_loss_backward"):
        check(_lib.load().mi_moe_aux_loss_backward(_ptr(logits), _ptr(loss_w.contiguous()), _ptr(grad), _ptr(d_logits),
                                                   T, E, _code(logits.dtype), _stream()))
    return d_logits


def scattered_experts(inputs: torch.Tensor, expert_weights: torch.Tensor, k: int,
                      sorted_expert_idxs: torch.Tensor, sorted_scattered_idxs: torch.Tensor,
                      expert_offsets: torch.Tensor, gates: torch.Tensor | None = None, grouped_in: bool = False,
                      grouped_out: bool = False, combine_tail: tuple | None = None) -> torch.Tensor:
    """Drop-in for the external ``scattered_experts`` (moe.py:91-101).

    ``expert_weights`` is the (E, in, out) view the reference passes (``weight.permute(0, 2, 1)``);
    ``sorted_expert_idxs`` is accepted for signature compatibility (the kernels derive the expert of
    a row from ``expert_offsets``).  With ``gates`` (T, k_g) the (L, out) result is contracted to
    (T, out); ``combine_tail`` = (shared, residual, residual_scale) is an extension handed on to
    :func:`combine`."""
    del sorted_expert_idxs
    if gates is not None and grouped_out:
        raise ValueError("gates need the output in flat-slot order (grouped_out=False)")
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (inputs, expert_weights, gates)):
        # like the reference's op this one is differentiable; the gradient lives in autograd.py
        if combine_tail is not None:
            raise ValueError("combine_tail is an inference-only fusion")
        from .autograd import ScatteredExperts

        return ScatteredExperts.apply(inputs, expert_weights.permute(0, 2, 1), k, _i32(sorted_scattered_idxs),
                                      _i32(expert_offsets), gates, grouped_in, grouped_out)
    w = _native_weight(expert_weights)
    out = scattered_gemm(inputs, w, k, sorted_scattered_idxs, expert_offsets, grouped_in, grouped_out)
    if combine_tail is not None and gates is None:
        raise ValueError("combine_tail needs gates")
    if gates is not None:
        out = combine(out, gates.to(out.dtype), *(combine_tail or ()))
    return out


def up_swiglu(x: torch.Tensor, w_fc: torch.Tensor, k: int, sorted_scattered_idxs: torch.Tensor,
              expert_offsets: torch.Tensor, cfg: int = -1, split_k: bool = True) -> torch.Tensor:
    """Up-projection with SwiGLU fused: x (T, H), w_fc (E, 2I, H) -> (L, I) in grouped order
    (``split_k`` as in scattered_gemm)."""
    _dev(x, w_fc, sorted_scattered_idxs, expert_offsets)
    _no_grad(x, w_fc)
    x = x.contiguous()
    w_fc = w_fc.contiguous()
    ss = _i32(sorted_scattered_idxs).contiguous()
    off = _i32(expert_offsets).contiguous()
    E, I2, H = w_fc.shape
    if x.shape[1] != H or w_fc.dtype != x.dtype or I2 % 2:
        raise ValueError("x must be (T, H), w_fc (E, 2I, H), same dtype")
    L = ss.numel()
    if x.shape[0] * k != L:
        raise ValueError("x must have L / k rows")
    act = torch.empty((L, I2 // 2), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    ws, ws_bytes = _gemm_workspace(x.device, H, x.dtype, split_k)
    with _stage("up_swiglu"):
        check(_gemm_or_slow(lambda c: lib.mi_moe_up_swiglu_ws(
            _ptr(x), _ptr(w_fc), _ptr(act), _ptr(ss), _ptr(off), L, H, I2 // 2, E, k, _code(x.dtype), c, _ptr(ws),
            ws_bytes, _stream()), cfg, H, I2 // 2, x.dtype, x.shape[0]))
    return act


def up_swiglu_keep(x: torch.Tensor, w_fc: torch.Tensor, k: int, sorted_scattered_idxs: torch.Tensor,
                   expert_offsets: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Up-projection for training: (act (L, I), h (L, 2I)) -- the activation and the pre-activation the backward
    needs.  One launch (mi_moe_up_swiglu_keep) where the persistent tile kernel takes the problem, else the grouped
    GEMM followed by the element-wise SwiGLU on the stored h; either way act is formed from the rounded h."""
    _dev(x, w_fc, sorted_scattered_idxs, expert_offsets)
    _no_grad(x, w_fc)
    x = x.contiguous()
    w_fc = w_fc.contiguous()
    ss = _i32(sorted_scattered_idxs).contiguous()
    off = _i32(expert_offsets).contiguous()
    E, I2, H = w_fc.shape
    if x.shape[1] != H or w_fc.dtype != x.dtype or I2 % 2:
        raise ValueError("x must be (T, H), w_fc (E, 2I, H), same dtype")
    L = ss.numel()
    if x.shape[0] * k != L:
        raise ValueError("x must have L / k rows")
    if x.dtype in (torch.float16, torch.bfloat16) and L > 0:
        lib = _lib.load()
        act = torch.empty((L, I2 // 2), dtype=x.dtype, device=x.device)
        h = torch.empty((L, I2), dtype=x.dtype, device=x.device)
        with _stage("up_swiglu"):
            rc = lib.mi_moe_up_swiglu_keep(_ptr(x), _ptr(w_fc), _ptr(act), _ptr(h), _ptr(ss), _ptr(off), L, H, I2 // 2,
                                           E, k, _code(x.dtype), _stream())
        if rc == 0:
            return act, h
        if rc not in (_lib.MI_MOE_EUNSUPPORTED, _lib.MI_MOE_EALIGN):
            check(rc)
    h = scattered_gemm(x, w_fc, k, ss, off, False, True)
    return swiglu_forward(h), h


def _fp8_unit_rows(glu: bool) -> int:
    return 16 if glu else 32


_FP8_SWIZZLE = None


def _fp8_swizzle_index(device):
    """(32, 1) row index and (32, 8) source-chunk index of the stage image: slot c of row t holds chunk
    c ^ (((t >> 1) & 1) | (((t >> 2) & 1) << 2))."""
    global _FP8_SWIZZLE
    if _FP8_SWIZZLE is None or _FP8_SWIZZLE[0].device != device:
        t = torch.arange(32, device=device)
        c = torch.arange(8, device=device)
        _FP8_SWIZZLE = (t[:, None], c[None, :] ^ (((t[:, None] >> 1) & 1) | (((t[:, None] >> 2) & 1) << 2)))
    return _FP8_SWIZZLE


def fp8_tile(w_q: torch.Tensor, glu: bool) -> torch.Tensor:
    """Row-major fp8 expert weights (E, out, in) -> the streamed-tile layout of include/mi_moe.h (a flat
    tensor): [expert][unit][K stage][32 rows][8 slots][16 bytes], units of 16 up + 16 gate channels (``glu``)
    or 32 channels, chunk slots pre-swizzled, channels past the last one zero.  Needs in % 128 == 0."""
    if w_q.dtype != torch.float8_e4m3fn or w_q.dim() != 3:
        raise TypeError("expected (E, out, in) torch.float8_e4m3fn")
    E, R, K = w_q.shape
    if K % 128 or (glu and R % 2):
        raise ValueError("the tile layout needs in % 128 == 0 (and an even row count for GLU weights)")
    b = w_q.contiguous().view(torch.uint8)
    ch = _fp8_unit_rows(glu)
    halves = b.chunk(2, dim=1) if glu else (b,)
    N = halves[0].shape[1]
    U = -(-N // ch)
    parts = []
    for h in halves:
        if U * ch != N:
            h = torch.cat([h, h.new_zeros(E, U * ch - N, K)], dim=1)
        parts.append(h.view(E, U, ch, K))
    unit = torch.cat(parts, dim=2) if glu else parts[0]                 # (E, U, 32, K)
    staged = unit.view(E, U, 32, K // 128, 8, 16).permute(0, 1, 3, 2, 4, 5)  # (E, U, stage, row, chunk, 16)
    rows, src = _fp8_swizzle_index(w_q.device)
    return staged[:, :, :, rows, src].contiguous().view(-1).view(torch.float8_e4m3fn)


def fp8_untile(tiled: torch.Tensor, E: int, out_rows: int, K: int, glu: bool) -> torch.Tensor:
    """Inverse of :func:`fp8_tile`: back to (E, out_rows, K) row-major."""
    ch = _fp8_unit_rows(glu)
    N = out_rows // 2 if glu else out_rows
    U = -(-N // ch)
    staged = tiled.view(torch.uint8).view(E, U, K // 128, 32, 8, 16)
    rows, src = _fp8_swizzle_index(tiled.device)
    unit = staged[:, :, :, rows, src].permute(0, 1, 3, 2, 4, 5).reshape(E, U, 32, K)   # the swizzle is an involution
    if glu:
        up = unit[:, :, :16].reshape(E, U * 16, K)[:, :N]
        gate = unit[:, :, 16:].reshape(E, U * 16, K)[:, :N]
        w = torch.cat([up, gate], dim=1)
    else:
        w = unit.reshape(E, U * 32, K)[:, :N]
    return w.contiguous().view(torch.float8_e4m3fn)


# Average rows per expert from which the fp8 calls widen the weights for the call and run the persistent 16-bit
# kernels instead of the library's own fp8 kernels (streaming for a few rows per expert, tiles that widen the bytes
# on their way into LDS beyond): the widening is one pass over all weights whatever the batch, and the persistent
# kernel is the faster GEMM.  Measured on the decode workload's shape (both projections): 384 rows per expert 1.34 ms
# on the fp8 tiles / 1.58 ms widened, 768 rows 2.27 / 2.23 ms, 1536 rows 4.16 / 3.55 ms.
FP8_DENSE_ROWS_PER_EXPERT = 768


def fp8_dequant(w_q: torch.Tensor, scale: torch.Tensor, in_features: int, glu: bool, dtype: torch.dtype) -> torch.Tensor:
    """e4m3fn expert weights, row-major (E, rows, in) or tiled (:func:`fp8_tile`), with (E, rows) fp32 scales ->
    (E, rows, in) weights of ``dtype`` (bf16 / fp16) = round(w * scale[:, :, None])."""
    _dev(w_q, scale)
    if w_q.dtype != torch.float8_e4m3fn or dtype not in (torch.bfloat16, torch.float16):
        raise TypeError("expected torch.float8_e4m3fn weights and a 16-bit result type")
    w_q = w_q.contiguous()
    scale = scale.to(torch.float32).contiguous()
    E, R = scale.shape
    K = int(in_features)
    tiled = w_q.dim() == 1
    lib = _lib.load()
    if (glu and R % 2) or K % 16:
        raise ValueError("shape mismatch")
    out_ch = R // 2 if glu else R
    if tiled:
        if w_q.numel() != lib.mi_moe_fp8_tiled_bytes(E, out_ch, K, int(glu)) or w_q.numel() == 0:
            raise ValueError("tiled weights do not match the scales and in_features")
    elif tuple(w_q.shape) != (E, R, K):
        raise ValueError("shape mismatch")
    w = torch.empty((E, R, K), dtype=dtype, device=w_q.device)
    with _stage("fp8_dequant"):
        check(lib.mi_moe_fp8_dequant(_ptr(w_q), _ptr(scale), _ptr(w), E, out_ch, K, int(glu), int(tiled), _code(dtype),
                                     _stream()))
    return w


def up_swiglu_fp8(x: torch.Tensor, w_fc_q: torch.Tensor, w_fc_scale: torch.Tensor, k: int,
                  sorted_scattered_idxs: torch.Tensor, expert_offsets: torch.Tensor,
                  widen: bool | None = None, cfg: int = -1) -> torch.Tensor:
    """As up_swiglu with e4m3fn weights and fp32 per-output-channel scales (E, 2I).  The weights are either
    row-major (E, 2I, H) or, as a flat tensor, in the layout of :func:`fp8_tile` (``glu=True``).  From
    FP8_DENSE_ROWS_PER_EXPERT rows per expert on average the weights are widened for the call and
    :func:`up_swiglu` runs on the copy (``widen``: True / False force either way).  Below that the library picks
    between its streaming kernels (decode: a few rows per expert) and the tile kernels that widen the fp8 bytes on
    their way into LDS (``cfg``: 0 / 1 force either, -1 picks by the batch)."""
    _dev(x, w_fc_q, w_fc_scale, sorted_scattered_idxs, expert_offsets)
    _no_grad(x)
    if w_fc_q.dtype != torch.float8_e4m3fn:
        raise TypeError("weights must be torch.float8_e4m3fn")
    x = x.contiguous()
    w_fc_q = w_fc_q.contiguous()
    scale = w_fc_scale.to(torch.float32).contiguous()
    ss = _i32(sorted_scattered_idxs).contiguous()
    off = _i32(expert_offsets).contiguous()
    E, I2 = scale.shape
    H = x.shape[1]
    L = ss.numel()
    tiled = w_fc_q.dim() == 1
    lib = _lib.load()
    if tiled:
        if w_fc_q.numel() != lib.mi_moe_fp8_tiled_bytes(E, I2 // 2, H, 1) or w_fc_q.numel() == 0:
            raise ValueError("tiled weights do not match (E, 2I) scales and the hidden size of x")
    elif tuple(w_fc_q.shape) != (E, I2, H):
        raise ValueError("shape mismatch")
    if x.shape[0] * k != L:
        raise ValueError("shape mismatch")
    if (L >= FP8_DENSE_ROWS_PER_EXPERT * E if widen is None else widen) and H % 16 == 0 and L > 0:
        return up_swiglu(x, fp8_dequant(w_fc_q, scale, H, True, x.dtype), k, ss, off)
    act = torch.empty((L, I2 // 2), dtype=x.dtype, device=x.device)
    with _stage("up_swiglu_fp8"):
        check(lib.mi_moe_up_swiglu_fp8_cfg(_ptr(x), _ptr(w_fc_q), _ptr(scale), _ptr(act), _ptr(ss), _ptr(off), L, H,
                                          I2 // 2, E, k, _code(x.dtype), int(tiled), int(cfg), _stream()))
    return act


def down_fp8(act: torch.Tensor, w_proj_q: torch.Tensor, w_proj_scale: torch.Tensor,
             sorted_scattered_idxs: torch.Tensor, expert_offsets: torch.Tensor,
             widen: bool | None = None, cfg: int = -1) -> torch.Tensor:
    """Down-projection with e4m3fn weights, row-major (E, H, I) or tiled (:func:`fp8_tile`, ``glu=False``):
    act (L, I) grouped -> (L, H) in flat-slot order (widened weights from FP8_DENSE_ROWS_PER_EXPERT rows per expert
    on, ``cfg`` below that, as in :func:`up_swiglu_fp8`)."""
    _dev(act, w_proj_q, w_proj_scale, sorted_scattered_idxs, expert_offsets)
    _no_grad(act)
    if w_proj_q.dtype != torch.float8_e4m3fn:
        raise TypeError("weights must be torch.float8_e4m3fn")
    act = act.contiguous()
    w_proj_q = w_proj_q.contiguous()
    scale = w_proj_scale.to(torch.float32).contiguous()
    ss = _i32(sorted_scattered_idxs).contiguous()
    off = _i32(expert_offsets).contiguous()
    E, H = scale.shape
    L, I = act.shape
    tiled = w_proj_q.dim() == 1
    lib = _lib.load()
    if tiled:
        if w_proj_q.numel() != lib.mi_moe_fp8_tiled_bytes(E, H, I, 0) or w_proj_q.numel() == 0:
            raise ValueError("tiled weights do not match (E, H) scales and the width of act")
    elif tuple(w_proj_q.shape) != (E, H, I):
        raise ValueError("shape mismatch")
    if ss.numel() != L:
        raise ValueError("shape mismatch")
    if (L >= FP8_DENSE_ROWS_PER_EXPERT * E if widen is None else widen) and I % 16 == 0 and L > 0:
        return scattered_gemm(act, fp8_dequant(w_proj_q, scale, I, False, act.dtype), 1, ss, off, True, False)
    o = torch.empty((L, H), dtype=act.dtype, device=act.device)
    with _stage("down_fp8"):
        check(lib.mi_moe_down_fp8_cfg(_ptr(act), _ptr(w_proj_q), _ptr(scale), _ptr(o), _ptr(ss), _ptr(off), L, I, H,
                                     E, _code(act.dtype), int(tiled), int(cfg), _stream()))
    return o
