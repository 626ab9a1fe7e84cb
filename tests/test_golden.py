"""The CPU oracle against the golden vectors in tests/golden/ (the reference's own known answers)."""
import json
import os

import pytest
import torch

from oracle import clt_oracle as orc

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


@pytest.mark.parametrize("case", GOLD["batchtopk"], ids=lambda c: c["source"])
def test_oracle_batchtopk(case):
    x = torch.tensor(case["x"])
    r = torch.tensor(case["ranking"]) if case["ranking"] is not None else None
    if "expected_mask" in case:
        assert torch.equal(orc.batchtopk_mask(x, case["k"], r), torch.tensor(case["expected_mask"]))
    if "expected_output" in case:
        assert torch.equal(orc.batchtopk_forward(x, float(case["k"]), r), torch.tensor(case["expected_output"]))


@pytest.mark.parametrize("case", GOLD["tokentopk"], ids=lambda c: c["source"])
def test_oracle_tokentopk(case):
    x = torch.tensor(case["x"])
    r = torch.tensor(case["ranking"]) if case["ranking"] is not None else None
    assert torch.equal(orc.tokentopk_mask(x, case["k"], r), torch.tensor(case["expected_mask"]))
    if "expected_output" in case:
        assert torch.equal(orc.tokentopk_forward(x, case["k"], r), torch.tensor(case["expected_output"]))


@pytest.mark.parametrize("case", GOLD["jumprelu"], ids=lambda c: c["source"])
def test_oracle_jumprelu(case):
    out = orc.jumprelu_forward(torch.tensor(case["x"]), torch.tensor([case["threshold"]]))
    assert torch.equal(out, torch.tensor(case["expected_output"]))


@pytest.mark.parametrize("case", GOLD["jumprelu_backward"], ids=lambda c: f"bw{c['bandwidth']}-x{c['input']}-t{c['threshold']}")
def test_oracle_jumprelu_backward(case):
    x = torch.tensor([case["input"]], dtype=torch.float64, requires_grad=True)
    thr = torch.tensor([case["threshold"]], dtype=torch.float64, requires_grad=True)
    out = orc.JumpReLUFunction.apply(x, thr, case["bandwidth"])
    out.backward(torch.tensor([case["grad_output"]], dtype=torch.float64))
    assert x.grad.item() == case["expected_grad_input"] * case["grad_output"]
    near = abs(case["input"] - case["threshold"]) <= case["bandwidth"] / 2.0
    want = (-case["input"] / case["bandwidth"]) * case["grad_output"] if near else 0.0
    assert thr.grad.item() == pytest.approx(want, abs=1e-12)
