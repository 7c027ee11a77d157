"""On-disk formats of the MoE layer's weights.

Two conversions, both pure functions over name -> tensor mappings (nothing here touches a GPU):

* Hugging Face Granite-MoE / Granite-MoE-Shared checkpoints <-> this module's state dict.  The HF layer
  keeps the fused up-projection as ``[gate ; up]`` (the first half goes through the activation), this
  module, like the reference, as ``[up ; gate]`` (``x[0] * act(x[1])``, activations/glu.py:42-43), so the
  two halves are swapped on the way in and out
  (lm_engine/hf_models/model_conversion/granitemoeshared.py:126-145 and 299-302).
* Tensor-parallel shards over the intermediate dimension.  ``c_fc`` is split per half -- rank r keeps
  rows ``[r*s, (r+1)*s)`` of the up half and of the gate half (s = I / world) -- and ``c_proj`` along its
  input dimension; the router is replicated.  The partial outputs of the ranks then simply add up
  (lm_engine/hf_models/models/gpt_base_TP/weights/shard.py:196-279).

Checkpoints are read with safetensors only: nothing in a file is executed.
"""

from __future__ import annotations

from typing import Iterable, Mapping

import torch

# module key -> HF key below "model.layers.{i}."; the bool says whether the GLU halves are swapped
_HF_KEYS = {
    "gate.weight": ("block_sparse_moe.router.layer.weight", None),
    "c_fc.weight": ("block_sparse_moe.input_linear.weight", 1),
    "c_proj.weight": ("block_sparse_moe.output_linear.weight", None),
    "c_fc_shared.weight": ("shared_mlp.input_linear.weight", 0),
    "c_proj_shared.weight": ("shared_mlp.output_linear.weight", None),
}
_SHARED_KEYS = ("c_fc_shared.weight", "c_proj_shared.weight")


def swap_glu_halves(weight: torch.Tensor, dim: int) -> torch.Tensor:
    """[a ; b] -> [b ; a] along ``dim`` (its own inverse)."""
    if weight.shape[dim] % 2:
        raise ValueError(f"dimension {dim} of a fused GLU weight must be even, got {weight.shape[dim]}")
    a, b = weight.chunk(2, dim=dim)
    return torch.cat([b, a], dim=dim)


def hf_layer_prefix(layer_idx: int) -> str:
    return f"model.layers.{layer_idx}."


def moe_state_dict_from_hf(hf_tensors: Mapping[str, torch.Tensor], layer_idx: int, glu: bool = True) -> dict:
    """State dict of one ``MoE`` module from the tensors of an HF Granite-MoE(-Shared) checkpoint.

    ``hf_tensors`` needs the layer's ``block_sparse_moe.*`` entries and, if the checkpoint has shared
    experts, ``shared_mlp.*``.  ``glu=False`` leaves the up-projections as they are (non-gated activations)."""
    prefix = hf_layer_prefix(layer_idx)
    out = {}
    for key, (hf_key, glu_dim) in _HF_KEYS.items():
        name = prefix + hf_key
        if name not in hf_tensors:
            if key in _SHARED_KEYS:
                continue
            raise KeyError(f"{name} is missing from the checkpoint")
        t = hf_tensors[name]
        out[key] = swap_glu_halves(t, glu_dim) if (glu and glu_dim is not None) else t
    if ("c_fc_shared.weight" in out) != ("c_proj_shared.weight" in out):
        raise KeyError(f"layer {layer_idx}: shared_mlp needs both input_linear and output_linear")
    return out


def moe_state_dict_to_hf(state_dict: Mapping[str, torch.Tensor], layer_idx: int, glu: bool = True) -> dict:
    """Inverse of :func:`moe_state_dict_from_hf`."""
    prefix = hf_layer_prefix(layer_idx)
    out = {}
    for key, (hf_key, glu_dim) in _HF_KEYS.items():
        if key not in state_dict:
            if key in _SHARED_KEYS:
                continue
            raise KeyError(f"{key} is missing from the state dict")
        t = state_dict[key]
        out[prefix + hf_key] = swap_glu_halves(t, glu_dim) if (glu and glu_dim is not None) else t
    return out


def load_moe_layer_from_safetensors(paths: str | Iterable[str], layer_idx: int, glu: bool = True,
                                    device: str | torch.device = "cpu") -> dict:
    """Reads one layer's MoE tensors from one or more ``.safetensors`` shards of an HF checkpoint
    (only that layer's tensors are materialised) and returns the module state dict."""
    from safetensors import safe_open

    if isinstance(paths, str):
        paths = [paths]
    wanted = {hf_layer_prefix(layer_idx) + hf_key for hf_key, _ in _HF_KEYS.values()}
    found = {}
    for path in paths:
        with safe_open(path, framework="pt", device=str(device)) as f:
            for name in f.keys():
                if name in wanted:
                    found[name] = f.get_tensor(name)
    return moe_state_dict_from_hf(found, layer_idx, glu=glu)


def save_moe_layer_to_safetensors(state_dict: Mapping[str, torch.Tensor], path: str, layer_idx: int,
                                  glu: bool = True) -> None:
    """Writes one layer's MoE tensors under their HF names."""
    from safetensors.torch import save_file

    save_file({k: v.contiguous() for k, v in moe_state_dict_to_hf(state_dict, layer_idx, glu=glu).items()}, path)


# ---- tensor-parallel shards over the intermediate dimension ----------------------------------------


def _split_halves(weight: torch.Tensor, dim: int, rank: int, world: int, glu: bool) -> torch.Tensor:
    n = weight.shape[dim]
    parts = 2 * world if glu else world
    if n % parts:
        raise ValueError(f"dimension {dim} ({n}) is not divisible by {parts}")
    s = n // parts
    first = weight.narrow(dim, rank * s, s)
    if not glu:
        return first.contiguous()
    second = weight.narrow(dim, (world + rank) * s, s)
    return torch.cat([first, second], dim=dim)


def tp_shard_moe_state_dict(state_dict: Mapping[str, torch.Tensor], rank: int, world: int, glu: bool = True) -> dict:
    """Rank ``rank``'s share of a MoE state dict: ``c_fc`` rows ``[r*s, (r+1)*s)`` of each GLU half,
    ``c_proj`` columns ``[r*s, (r+1)*s)``, router replicated (same for the shared experts)."""
    if not 0 <= rank < world:
        raise ValueError("rank out of range")
    out = {"gate.weight": state_dict["gate.weight"]}
    out["c_fc.weight"] = _split_halves(state_dict["c_fc.weight"], 1, rank, world, glu)
    out["c_proj.weight"] = _split_halves(state_dict["c_proj.weight"], 2, rank, world, False)
    if "c_fc_shared.weight" in state_dict:
        out["c_fc_shared.weight"] = _split_halves(state_dict["c_fc_shared.weight"], 0, rank, world, glu)
        out["c_proj_shared.weight"] = _split_halves(state_dict["c_proj_shared.weight"], 1, rank, world, False)
    return out


def _join_halves(parts: list, dim: int, glu: bool) -> torch.Tensor:
    if not glu:
        return torch.cat(parts, dim=dim)
    firsts, seconds = zip(*(p.chunk(2, dim=dim) for p in parts))
    return torch.cat(list(firsts) + list(seconds), dim=dim)


def tp_unshard_moe_state_dicts(shards: list, glu: bool = True) -> dict:
    """Inverse of :func:`tp_shard_moe_state_dict` given the shards in rank order."""
    if not shards:
        raise ValueError("no shards")
    out = {"gate.weight": shards[0]["gate.weight"]}
    out["c_fc.weight"] = _join_halves([s["c_fc.weight"] for s in shards], 1, glu)
    out["c_proj.weight"] = _join_halves([s["c_proj.weight"] for s in shards], 2, False)
    if "c_fc_shared.weight" in shards[0]:
        out["c_fc_shared.weight"] = _join_halves([s["c_fc_shared.weight"] for s in shards], 0, glu)
        out["c_proj_shared.weight"] = _join_halves([s["c_proj_shared.weight"] for s in shards], 1, False)
    return out
