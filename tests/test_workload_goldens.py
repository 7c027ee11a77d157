"""The seeded workloads must be the tensors tests/golden/workloads.json was written for.

Every parity result on the five benchmark configurations starts from ``oracle.make_inputs``; a drift of torch's
CPU generator between machines or versions would silently change all of them.  The SHA-256 of every generated
tensor is therefore pinned, and the oracle's routing on those inputs is re-derived and compared with the stored
histogram and first-token routing (pure CPU, no kernel involved)."""

import pytest
import torch

from oracle import moe_oracle as oracle

from _parity import tensor_sha256, workload_goldens, workload_inputs

NAMES = list(oracle.WORKLOADS)


def test_goldens_cover_every_workload():
    assert sorted(workload_goldens()) == sorted(NAMES)
    for name, rec in workload_goldens().items():
        w = oracle.WORKLOADS[name]
        assert (rec["seed"], rec["T"], rec["H"], rec["E"], rec["k"], rec["I"]) == (w.seed, w.T, w.H, w.E, w.k, w.I)
        assert sum(rec["routing"]["histogram"]) == w.T * w.k
        assert len(rec["output"]["values"]) == len(rec["output"]["positions"]) == 64


@pytest.mark.parametrize("name", NAMES)
def test_generated_inputs_match_recorded_hashes(name):
    rec = workload_goldens()[name]
    inputs = workload_inputs(name)
    got = {n: tensor_sha256(t) for n, t in inputs.items() if t is not None}
    assert got == rec["sha256"], "the CPU generator no longer produces the recorded tensors"


@pytest.mark.parametrize("name", NAMES)
def test_oracle_routing_matches_recorded_routing(name):
    rec = workload_goldens()[name]["routing"]
    w = oracle.WORKLOADS[name]
    inputs = workload_inputs(name)
    _, gates, experts = oracle.route(inputs["x"], inputs["gate_w"], w.k, bias=inputs["bias"])
    n = len(rec["experts_first_tokens"])
    assert experts[:n].tolist() == rec["experts_first_tokens"]
    assert torch.bincount(experts.flatten(), minlength=w.E).tolist() == rec["histogram"]
    torch.testing.assert_close(gates[:n].float(), torch.tensor(rec["gates_first_tokens"]), rtol=0, atol=0)
