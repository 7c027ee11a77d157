"""The HIP path on committed golden data.

* tests/golden/workloads.json (written by tests/golden/make_workload_goldens.py FROM THE ORACLE, on inputs that
  oracle.make_inputs draws again here): the five benchmark / parity workloads at full size; the device's routing
  must reproduce the recorded histogram and first-token routing exactly and the layer output the recorded slice and
  checksums of the fp32 result.  This is the oracle's answer frozen -- it guards against drift of the oracle, the
  generator or the kernels between machines and versions; it is not evidence independent of the oracle.
* The two .npz files below ARE independent of oracle/: neither their inputs nor their expected outputs pass
  through it.
* tests/golden/granitemoe_h32_e8_k{2,8}.npz (written by tests/golden/make_golden.py from transformers'
  GraniteMoeMoE, which the reference asserts its eager branch equals:
  tests/hf_models/single_gpu/model_conversion_test.py:60-103): loaded into the module directly and through a
  Hugging Face layout safetensors file (lm_engine/hf_models/model_conversion/granitemoeshared.py:126-145, 299-302).
"""

import glob
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as oracle

from _parity import GOLDEN_DIR, assert_close_scaled, workload_goldens, workload_inputs

pytestmark = pytest.mark.gpu

NPZ = sorted(glob.glob(os.path.join(GOLDEN_DIR, "granitemoe_*.npz")))


def _module(H, I, E, k, dtype, device, padding_free=True):
    from dolomite_engine_amd import MoE

    return MoE(hidden_size=H, intermediate_size=I, shared_intermediate_size=None, num_experts=E,
               num_experts_per_tok=k, activation_function="swiglu", add_bias=False, dropout=0.0,
               init_method="normal", initializer_range=0.02, m_width=None, num_layers=1,
               use_padding_free_transformer=padding_free).to(dtype).to(device).eval()


@pytest.mark.parametrize("name", list(oracle.WORKLOADS))
def test_workload_golden_on_device(device, name):
    from dolomite_engine_amd import Kernel, enable_kernels, ops

    w = oracle.WORKLOADS[name]
    rec = workload_goldens()[name]
    inputs = workload_inputs(name)
    m = _module(w.H, w.I, w.E, w.k, w.dtype, device)
    with torch.no_grad():
        m.gate.weight.copy_(inputs["gate_w"])
        if w.fp8:
            m.c_fc.set_fp8_weight(inputs["w_fc"].to(device), inputs["fc_scale"].to(device), w.dtype, tiled=True, glu=True)
            m.c_proj.set_fp8_weight(inputs["w_proj"].to(device), inputs["proj_scale"].to(device), w.dtype, tiled=True,
                                    glu=False)
        else:
            m.c_fc.weight.copy_(inputs["w_fc"])
            m.c_proj.weight.copy_(inputs["w_proj"])
    if inputs["bias"] is not None:
        m.router_logit_bias = inputs["bias"].to(device)
    x = inputs["x"].to(device)
    print(f"workload golden {name}", flush=True)
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        y = m(x)
        _, gates, idx = m._compute_routing_weights(x)
        _, _, off = ops.sort_bin(idx, w.E)
    # routing: integer work, exact
    n = len(rec["routing"]["experts_first_tokens"])
    assert idx[:n].cpu().tolist() == rec["routing"]["experts_first_tokens"]
    counts = torch.diff(off.cpu().long(), prepend=torch.zeros(1, dtype=torch.long))
    moved = (counts - torch.tensor(rec["routing"]["histogram"])).abs().sum().item() // 2
    print(f"  slots routed differently from the recorded histogram: {moved}", flush=True)
    assert moved == 0
    step = {torch.float32: 1e-6, torch.bfloat16: 4e-3, torch.float16: 5e-4}[w.dtype]  # half a unit in the last place
    torch.testing.assert_close(gates[:n].cpu().float(), torch.tensor(rec["routing"]["gates_first_tokens"]), rtol=step,
                               atol=step)
    # output: recorded slice of the fp32 result, and its checksums
    yc = y.cpu().float()
    pos = torch.tensor(rec["output"]["positions"])
    got = yc[pos[:, 0], pos[:, 1]]
    want = torch.tensor(rec["output"]["values"])
    tol = dict(rtol=1e-3, atol=2e-4) if w.dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    assert_close_scaled(got, want, w.dtype, what=f"{name} slice", **tol)
    abs_sum = yc.double().abs().sum().item()
    assert abs(abs_sum - rec["output"]["abs_sum"]) <= 2e-3 * rec["output"]["abs_sum"]
    assert abs(yc.double().sum().item() - rec["output"]["sum"]) <= 1e-3 * rec["output"]["abs_sum"]
    assert abs(yc.abs().max().item() - rec["output"]["abs_max"]) <= 2e-2 * rec["output"]["abs_max"]


def _load_npz(path):
    z = np.load(path)
    return {n: torch.from_numpy(z[n]) for n in ("x", "gate_w", "w_fc", "w_proj", "topk_idx", "gates", "y")}, int(z["k"])


def _check_against_npz(m, g, k, dtype, device):
    from dolomite_engine_amd import Kernel, enable_kernels

    x = g["x"].to(dtype).to(device)
    with torch.no_grad(), enable_kernels([Kernel.scattermoe]):
        y = m(x.unsqueeze(0)).squeeze(0)
        _, gates, idx = m._compute_routing_weights(x)
    if dtype == torch.float32:
        assert torch.equal(idx.cpu().long(), g["topk_idx"])
        torch.testing.assert_close(gates.cpu(), g["gates"], rtol=1e-5, atol=1e-6)
        # the reference's fp32 bar for this path (tests/hf_models/single_gpu/scattermoe_test.py:38-42)
        assert_close_scaled(y, g["y"], dtype, rtol=1e-3, atol=2e-4, what="fp32")
        return
    # 16-bit: rounding x and the gate weights moves logits by about one part in 2^8, which can swap two experts
    # of nearly equal logit.  Rows that select the recorded experts (as a set) are compared; most rows must.
    same = (idx.cpu().long().sort(dim=1).values == g["topk_idx"].sort(dim=1).values).all(dim=1)
    print(f"  rows with the recorded expert set: {int(same.sum())} of {same.numel()}", flush=True)
    assert same.sum().item() >= 0.8 * same.numel()
    # the recorded output comes from the unrounded fp32 tensors: rounding x and the three weight tensors to 16 bits
    # adds to the kernel's own rounding, so the scaled bounds are three times those of a same-input comparison
    lim = {torch.bfloat16: 2.5e-2, torch.float16: 4e-3}[dtype]
    assert_close_scaled(y[same.to(device)], g["y"][same], dtype, rtol=2e-2, atol=2e-2, what=str(dtype),
                        rel_to_max=lim, rel_rms_limit=lim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("path", NPZ, ids=[os.path.basename(p) for p in NPZ])
def test_independent_golden_through_hip_path(device, path, dtype):
    g, k = _load_npz(path)
    E, I2, H = g["w_fc"].shape
    m = _module(H, I2 // 2, E, k, dtype, device, padding_free=False)
    with torch.no_grad():
        m.gate.weight.copy_(g["gate_w"])
        m.c_fc.weight.copy_(g["w_fc"])
        m.c_proj.weight.copy_(g["w_proj"])
    print(f"npz golden {os.path.basename(path)} {dtype}", flush=True)
    _check_against_npz(m, g, k, dtype, device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("path", NPZ, ids=[os.path.basename(p) for p in NPZ])
def test_hf_checkpoint_through_hip_path(device, path, dtype, tmp_path):
    """An HF-layout safetensors file ([gate ; up] fused up-projection, HF tensor names) written here by hand,
    read with checkpoint.load_moe_layer_from_safetensors, loaded with load_state_dict and run on the kernels."""
    from safetensors.torch import save_file

    from dolomite_engine_amd import checkpoint

    g, k = _load_npz(path)
    E, I2, H = g["w_fc"].shape
    up, gate = g["w_fc"].chunk(2, dim=1)
    layer = 3
    prefix = f"model.layers.{layer}.block_sparse_moe."
    f = str(tmp_path / "layer.safetensors")
    save_file({
        prefix + "router.layer.weight": g["gate_w"].to(dtype).contiguous(),
        prefix + "input_linear.weight": torch.cat([gate, up], dim=1).to(dtype).contiguous(),   # HF order
        prefix + "output_linear.weight": g["w_proj"].to(dtype).contiguous(),
        "model.layers.2.block_sparse_moe.router.layer.weight": torch.zeros(E, H, dtype=dtype),  # another layer's
    }, f)
    sd = checkpoint.load_moe_layer_from_safetensors(f, layer)
    m = _module(H, I2 // 2, E, k, dtype, device, padding_free=False)
    m.load_state_dict(sd)  # strict: exactly the module's keys, in the module's shapes
    print(f"checkpoint golden {os.path.basename(path)} {dtype}", flush=True)
    _check_against_npz(m, g, k, dtype, device)
