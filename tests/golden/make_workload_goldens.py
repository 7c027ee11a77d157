"""Writes tests/golden/workloads.json: what the five seeded benchmark / parity workloads must look like.

For every workload of ``oracle.WORKLOADS`` the file records

* the seed and shape, and the SHA-256 of the bytes of every generated tensor (x, gate weight, both expert weight
  tensors, the Zipf logit bias, the fp8 scales), so that a drift of the CPU random generator between machines or
  torch versions is noticed instead of silently changing every parity result;
* the routing of the CPU oracle on its own logits: the per-expert slot histogram, the experts and gates of the
  first 64 tokens, the share of tokens with a tie inside the top-(k+1) logits;
* the layer output of the fp32 oracle: sum, sum of magnitudes, largest magnitude, and the values at 64 fixed
  positions.

The reference holds no stored vectors for this path (its tests compare two implementations on seeded inputs:
tests/hf_models/single_gpu/scattermoe_test.py:15-48, seed 1234; tests/hf_models/test_common.py:96-170), so these
are this repository's own, produced by the pinned oracle on this script's inputs.

    python tests/golden/make_workload_goldens.py        # a few minutes of CPU, about 30 GB of memory at the peak
"""

import hashlib
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import moe_oracle as oracle  # noqa: E402

OUT = os.path.join(HERE, "workloads.json")
N_ROUTING_TOKENS = 64
N_SLICE = 64


def tensor_sha256(t: torch.Tensor) -> str:
    """SHA-256 of the tensor's bytes in row-major order (any dtype, including bf16 and fp8)."""
    t = t.contiguous()
    raw = t.view(torch.uint8) if t.element_size() == 1 else t.view(-1).view(torch.uint8)
    return hashlib.sha256(raw.numpy().tobytes()).hexdigest()


def slice_positions(T: int, H: int, n: int = N_SLICE) -> list:
    """n fixed (token, column) positions spread over the output by two coprime strides."""
    return [((i * 2654435761) % T, (i * 40503 + 7) % H) for i in range(n)]


def describe(w: oracle.Workload) -> dict:
    inputs = oracle.make_inputs(w)
    rec = {
        "seed": w.seed, "T": w.T, "H": w.H, "E": w.E, "k": w.k, "I": w.I, "dtype": str(w.dtype).replace("torch.", ""),
        "sha256": {name: tensor_sha256(t) for name, t in inputs.items() if t is not None},
    }
    out = oracle.moe_forward(inputs["x"], inputs["gate_w"], inputs["w_fc"], inputs["w_proj"], w.k, bias=inputs["bias"],
                             w_fc_scale=inputs["fc_scale"], w_proj_scale=inputs["proj_scale"])
    counts = torch.bincount(out.experts.flatten(), minlength=w.E)
    # rows whose routing a one-step rounding difference of the logits could change: a tie inside the top-(k+1)
    srt = out.logits.float().sort(dim=-1, descending=True).values[:, : min(w.k + 1, w.E)]
    tied = (srt.diff(dim=-1) == 0).any(dim=-1).float().mean().item()
    n = min(N_ROUTING_TOKENS, w.T)
    pos = slice_positions(w.T, w.H)
    y = out.y.double()
    rec["routing"] = {
        "histogram": counts.tolist(),
        "experts_first_tokens": out.experts[:n].tolist(),
        "gates_first_tokens": out.gates[:n].float().tolist(),
        "rows_with_tie_in_top_k_plus_1": tied,
    }
    rec["output"] = {
        "sum": y.sum().item(), "abs_sum": y.abs().sum().item(), "abs_max": y.abs().max().item(),
        "positions": pos, "values": [out.y[t, c].item() for t, c in pos],
    }
    return rec


def main() -> None:
    torch.set_num_threads(os.cpu_count() or 1)
    doc = {"torch": torch.__version__, "workloads": {}}
    for name, w in oracle.WORKLOADS.items():
        print("workload", name, flush=True)
        doc["workloads"][name] = describe(w)
    with open(OUT, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    print("wrote", OUT)


if __name__ == "__main__":
    main()
