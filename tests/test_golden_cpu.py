"""The oracle reproduces the committed golden vectors (guards the oracle against drift)."""
import pytest
import torch

from oracle import attention_oracle as O
from tests import golden_cases

CASES = golden_cases.load()


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_golden(name):
    case = CASES[name]
    out = O.reference_layer(case["q"], case["k"], case["v"], **golden_cases.oracle_kwargs(case, O))
    assert out.shape == case["out"].shape
    assert (out - case["out"].double()).abs().max() < 2e-6  # stored as float32
    assert torch.isfinite(case["out"]).all()
