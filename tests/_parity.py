"""Shared pieces of the parity tests: cached workload inputs and a comparison that cannot pass vacuously."""

import functools
import hashlib
import json
import os

import torch

from oracle import moe_oracle as oracle

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# largest error relative to the LARGEST reference entry that a correct 16-bit kernel path leaves against the fp32
# oracle (three roundings of intermediates of about the output's size), and the same for the root-mean-square error
REL_TO_MAX = {torch.bfloat16: 1e-2, torch.float16: 2e-3, torch.float32: 2e-5}
REL_RMS = {torch.bfloat16: 8e-3, torch.float16: 1.5e-3, torch.float32: 1e-5}


@functools.lru_cache(maxsize=None)
def workload_inputs(name: str, T: int | None = None) -> dict:
    """oracle.make_inputs, computed once per test session (the big workloads take seconds to draw)."""
    return oracle.make_inputs(oracle.WORKLOADS[name], T=T)


@functools.lru_cache(maxsize=1)
def workload_goldens() -> dict:
    with open(os.path.join(GOLDEN_DIR, "workloads.json")) as f:
        return json.load(f)["workloads"]


def tensor_sha256(t: torch.Tensor) -> str:
    """SHA-256 of a tensor's bytes in row-major order (the definition tests/golden/make_workload_goldens.py uses)."""
    t = t.contiguous()
    raw = t.view(torch.uint8) if t.element_size() == 1 else t.view(-1).view(torch.uint8)
    return hashlib.sha256(raw.numpy().tobytes()).hexdigest()


def assert_close_scaled(got: torch.Tensor, ref: torch.Tensor, dtype: torch.dtype, rtol: float, atol: float,
                        what: str = "", rel_to_max: float | None = None, rel_rms_limit: float | None = None) -> None:
    """The stated tolerance (rtol / atol, element-wise) AND bounds that scale with the output, so that small
    outputs cannot hide inside an absolute tolerance: the reference must be far from zero compared with what is
    allowed, the largest error is bounded relative to the largest reference entry, and so is the RMS error."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    ref_max = ref.abs().max().item()
    assert ref_max > 0 and torch.isfinite(got).all(), what
    err = (got - ref).abs()
    rel_max = err.max().item() / ref_max
    rel_rms = (err.pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30)).item()
    print(f"  {what} max|ref| {ref_max:.3e}  max err / max|ref| {rel_max:.2e}  rms err / rms ref {rel_rms:.2e}", flush=True)
    assert rel_max <= (rel_to_max or REL_TO_MAX[dtype]), \
        f"{what}: largest error is {rel_max:.2e} of the largest reference entry"
    assert rel_rms <= (rel_rms_limit or REL_RMS[dtype]), f"{what}: rms error is {rel_rms:.2e} of the rms of the reference"
    assert got.abs().max().item() > 0.5 * ref_max, f"{what}: output is far smaller than the reference"
    torch.testing.assert_close(got, ref, rtol=rtol, atol=atol)
