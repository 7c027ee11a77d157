"""GPU parity of the element-wise backward kernels against fp32 formulas evaluated with torch autograd on the CPU.

The expected values come from differentiating the forward definitions (``up * silu(gate)``,
activations/glu.py:42-43, and the gate-weighted sum of moe.py:282-290) with autograd in fp32, not from a
retyped derivative; results are 16-bit so the comparison is at the rounding of the output dtype.
"""

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _ops():
    from dolomite_engine_amd import ops

    return ops


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,I", [(1, 8), (37, 64), (513, 512), (4099, 1408)])
@pytest.mark.parametrize("scaled", [False, True])
def test_swiglu_backward(device, dtype, L, I, scaled):
    g = torch.Generator().manual_seed(L * 31 + I)
    h = (torch.randn(L, 2 * I, generator=g) * 2).to(dtype)
    d_act = torch.randn(L, I, generator=g).to(dtype)
    s = torch.rand(L, generator=g).to(dtype) if scaled else None

    hf = h.float().requires_grad_(True)
    a = hf[:, :I] * F.silu(hf[:, I:])
    upstream = d_act.float() * (s.float().unsqueeze(-1) if scaled else 1.0)
    a.backward(upstream)

    got = _ops().swiglu_backward(h.to(device), d_act.to(device), None if s is None else s.to(device))
    assert got.dtype == dtype and tuple(got.shape) == (L, 2 * I)
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    torch.testing.assert_close(got.cpu().float(), hf.grad, rtol=2 * eps, atol=1e-6)


def test_swiglu_backward_empty_and_errors(device):
    ops = _ops()
    out = ops.swiglu_backward(torch.empty(0, 32, device=device, dtype=torch.bfloat16),
                              torch.empty(0, 16, device=device, dtype=torch.bfloat16))
    assert tuple(out.shape) == (0, 32)
    with pytest.raises(ValueError):
        ops.swiglu_backward(torch.zeros(4, 30, device=device, dtype=torch.bfloat16),
                            torch.zeros(4, 16, device=device, dtype=torch.bfloat16))
    from dolomite_engine_amd._lib import MiMoeError

    with pytest.raises(MiMoeError):  # fp32 is not a dtype of this kernel
        ops.swiglu_backward(torch.zeros(4, 32, device=device), torch.zeros(4, 16, device=device))
    with pytest.raises(MiMoeError):  # I % 8 != 0
        ops.swiglu_backward(torch.zeros(4, 24, device=device, dtype=torch.bfloat16),
                            torch.zeros(4, 12, device=device, dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,H", [(1, 1, 8), (5, 2, 64), (300, 8, 1536), (64, 6, 4096), (1027, 2, 520)])
def test_combine_grad_gates(device, dtype, T, k, H):
    g = torch.Generator().manual_seed(T + k + H)
    o = torch.randn(T * k, H, generator=g).to(dtype)
    dy = torch.randn(T, H, generator=g).to(dtype)
    gates = torch.rand(T, k, generator=g).requires_grad_(True)
    y = (gates.unsqueeze(-1) * o.float().view(T, k, H)).sum(dim=1)
    y.backward(dy.float())

    got = _ops().combine_grad_gates(o.to(device), dy.to(device), k)
    assert got.dtype == dtype and tuple(got.shape) == (T, k)
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    # an fp32 dot product of H terms rounded once; the absolute term covers cancellation
    torch.testing.assert_close(got.cpu().float(), gates.grad, rtol=2 * eps, atol=1e-4 * H ** 0.5)
