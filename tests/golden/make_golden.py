"""Writes the golden vectors of tests/golden/*.npz.

The expected outputs do NOT come from this repository's oracle: they are computed by an independent
implementation of the same layer, transformers' ``GraniteMoeMoE`` (router: fp32 logits -> top-k ->
softmax over the k logits; experts: per-expert loop with a [gate ; up] fused weight).  The reference
asserts that its eager MoE branch equals exactly this module after swapping the two halves of the
up-projection weight (tests/hf_models/single_gpu/model_conversion_test.py:60-103 with
lm_engine/hf_models/model_conversion/granitemoeshared.py:126-136, 299-302), so a vector that holds for
it holds for the reference's eager branch.

Shapes follow the reference's own scattermoe test (hidden 32, 8 experts, intermediate 4*32,
15 tokens; tests/hf_models/test_common.py:96-170) with top-k 2 and 8.

    python tests/golden/make_golden.py          # rewrites the .npz files next to this script
"""

import os

import numpy as np
import torch
from transformers.models.granitemoe.configuration_granitemoe import GraniteMoeConfig
from transformers.models.granitemoe.modeling_granitemoe import GraniteMoeMoE

HERE = os.path.dirname(os.path.abspath(__file__))


def make_case(name: str, T: int, H: int, E: int, k: int, I: int, seed: int) -> None:
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g)
    gate_w = torch.randn(E, H, generator=g) * 0.5      # well separated logits: no ties in fp32
    w_fc = torch.randn(E, 2 * I, H, generator=g) * 0.1   # [up ; gate] rows, the reference's layout
    w_proj = torch.randn(E, H, I, generator=g) * 0.1

    cfg = GraniteMoeConfig(hidden_size=H, intermediate_size=I, num_local_experts=E, num_experts_per_tok=k,
                           hidden_act="silu")
    hf = GraniteMoeMoE(cfg).eval()
    with torch.no_grad():
        hf.router.weight.copy_(gate_w)
        up, gate = w_fc.chunk(2, dim=1)
        hf.experts.gate_up_proj.copy_(torch.cat([gate, up], dim=1))  # transformers keeps [gate ; up]
        hf.experts.down_proj.copy_(w_proj)
        idx, weights, logits = hf.router(x)
        y = hf(x.unsqueeze(0)).squeeze(0)
    np.savez(os.path.join(HERE, name + ".npz"), x=x.numpy(), gate_w=gate_w.numpy(), w_fc=w_fc.numpy(),
             w_proj=w_proj.numpy(), k=np.int64(k), logits=logits.numpy(), topk_idx=idx.numpy(),
             gates=weights.numpy(), y=y.numpy())
    print(name, "written; |y| max", float(y.abs().max()))


if __name__ == "__main__":
    make_case("granitemoe_h32_e8_k2", T=15, H=32, E=8, k=2, I=128, seed=1234)
    make_case("granitemoe_h32_e8_k8", T=15, H=32, E=8, k=8, I=128, seed=1235)
