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
