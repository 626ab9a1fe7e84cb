"""The HIP path (autograd Functions over the C ABI) against the golden vectors in tests/golden/."""
import json
import os

import pytest
import torch

from crosslayer_coding_amd.activations import BatchTopK, JumpReLU, TokenTopK

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", GOLD["batchtopk"], ids=lambda c: c["source"])
def test_hip_batchtopk(dev, case, dtype):
    x = torch.tensor(case["x"], device=dev).to(dtype)
    r = torch.tensor(case["ranking"], device=dev).to(dtype) if case["ranking"] is not None else None
    if "expected_mask" in case:
        mask = BatchTopK._compute_mask(x, case["k"], r)
        assert mask.dtype == torch.bool and torch.equal(mask.cpu(), torch.tensor(case["expected_mask"]))
    if "expected_output" in case:
        out = BatchTopK.apply(x, float(case["k"]), True, r)
        assert torch.equal(out.float().cpu(), torch.tensor(case["expected_output"]))


@pytest.mark.parametrize("case", GOLD["tokentopk"], ids=lambda c: c["source"])
def test_hip_tokentopk(dev, case):
    x = torch.tensor(case["x"], device=dev)
    r = torch.tensor(case["ranking"], device=dev) if case["ranking"] is not None else None
    assert torch.equal(TokenTopK._compute_mask(x, case["k"], r).cpu(), torch.tensor(case["expected_mask"]))
    if "expected_output" in case:
        assert torch.equal(TokenTopK.apply(x, case["k"], True, r).cpu(), torch.tensor(case["expected_output"]))


@pytest.mark.parametrize("case", GOLD["jumprelu"], ids=lambda c: c["source"])
def test_hip_jumprelu(dev, case):
    x = torch.tensor(case["x"], device=dev)
    out = JumpReLU.apply(x, torch.tensor([case["threshold"]], device=dev), 1.0)
    assert torch.equal(out.cpu(), torch.tensor(case["expected_output"]))
