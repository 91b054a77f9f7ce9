"""Oracle suffix operators against the reference's known-answer cases and its round-trip / validation tests
(test/auto_test/test_jagged_suffix.py:33-83, 130-182, 249-285)."""

import pytest
import torch

import oracle
from golden_cases import SUFFIX


@pytest.mark.parametrize("case", SUFFIX, ids=[c["name"] for c in SUFFIX])
def test_known_answers_and_round_trip(case):
    jag = oracle.JaggedTokens(tokens=case["tokens"], weight=case["weight"], offset=case["offset"])
    got = oracle.add_suffix(jag, case["suffix"])
    assert torch.equal(got.tokens, case["out"])
    assert torch.equal(got.weight, case["out_weight"])
    assert torch.equal(got.offset, case["out_offset"])
    back, suffix = oracle.split_suffix(got, case["suffix"].shape[1])
    assert torch.equal(back.tokens, jag.tokens) and torch.equal(back.weight, jag.weight)
    assert torch.equal(back.offset, jag.offset) and torch.equal(suffix, case["suffix"])


def test_validation_messages():
    jag = oracle.JaggedTokens(tokens=torch.randn(1, 6, 4), weight=torch.ones(6), offset=torch.tensor([0, 3, 6]))
    with pytest.raises(ValueError, match="suffix batch dim"):
        oracle.add_suffix(jag, torch.randn(3, 2, 4))
    short = oracle.JaggedTokens(tokens=torch.randn(1, 6, 4), weight=torch.ones(6), offset=torch.tensor([0, 1, 6]))
    with pytest.raises(ValueError, match="exceeds the length"):
        oracle.split_suffix(short, 2)
    with pytest.raises(ValueError, match="Cannot strip"):
        oracle.split_suffix(oracle.JaggedTokens(tokens=torch.randn(1, 4, 4), weight=torch.ones(4),
                                                offset=torch.tensor([0, 2, 4])), 100)
