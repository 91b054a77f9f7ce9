"""HIP suffix operators (JaggedTokens.add_suffix / split_suffix) through the C ABI: the reference's known-answer
cases, its round-trip and invariant tests (test/auto_test/test_jagged_suffix.py:33-83, 130-246) and its validation
messages (:249-285).  Row copies: bit-exact."""

import pytest
import torch

import oracle
from come_amd.interface import JaggedTokens
from golden_cases import SUFFIX

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("case", SUFFIX, ids=[c["name"] for c in SUFFIX])
def test_known_answers_and_round_trip(case):
    jag = JaggedTokens(tokens=case["tokens"].to(DEV), weight=case["weight"].to(DEV), offset=case["offset"].to(DEV))
    got = jag.add_suffix(case["suffix"].to(DEV))
    assert torch.equal(got.tokens.cpu(), case["out"])
    assert torch.equal(got.weight.cpu(), case["out_weight"])
    assert torch.equal(got.offset.cpu(), case["out_offset"]) and got.offset.dtype == torch.int64
    back, suffix = got.split_suffix(case["suffix"].shape[1])
    assert torch.equal(back.tokens.cpu(), case["tokens"]) and torch.equal(back.weight.cpu(), case["weight"])
    assert torch.equal(back.offset.cpu(), case["offset"]) and torch.equal(suffix.cpu(), case["suffix"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("M,T,C,lo,hi", [(1, 1, 8, 1, 1), (1, 4, 16, 5, 20), (4, 1, 32, 1, 10), (4, 3, 64, 2, 15),
                                         (8, 2, 16, 3, 30), (16, 5, 128, 1, 50), (32, 1, 8, 10, 10), (5, 2, 3, 0, 6),
                                         (32, 5, 1024, 300, 900)])
def test_random_against_oracle_and_round_trip(M, T, C, lo, hi, dtype):
    g = torch.Generator().manual_seed(M * 100 + T)
    lengths = torch.randint(lo, hi + 1, (M,), generator=g)
    P = int(lengths.sum())
    offset = torch.cat((torch.zeros(1, dtype=torch.long), lengths.cumsum(0)))
    tokens = torch.randn(1, P, C, generator=g).to(dtype)
    weight = torch.randint(1, 5, (P,), generator=g).float()
    suffix = torch.randn(M, T, C, generator=g).to(dtype)
    want = oracle.add_suffix(oracle.JaggedTokens(tokens=tokens, weight=weight, offset=offset), suffix)
    jag = JaggedTokens(tokens=tokens.to(DEV), weight=weight.to(DEV), offset=offset.to(DEV))
    got = jag.add_suffix(suffix.to(DEV))
    assert torch.equal(got.tokens.cpu(), want.tokens) and torch.equal(got.weight.cpu(), want.weight)
    assert torch.equal(got.offset.cpu(), want.offset)
    new_lens = got.offset[1:] - got.offset[:-1]
    assert torch.equal(new_lens.cpu(), lengths + T) and int(got.offset[-1]) == P + M * T
    back, tail = got.split_suffix(T)
    assert torch.equal(back.tokens.cpu(), tokens) and torch.equal(back.weight.cpu(), weight)
    assert torch.equal(back.offset.cpu(), offset) and torch.equal(tail.cpu(), suffix)


def test_validation_messages():
    jag = JaggedTokens(tokens=torch.randn(1, 6, 4, device=DEV), weight=torch.ones(6, device=DEV),
                       offset=torch.tensor([0, 3, 6], device=DEV))
    with pytest.raises(ValueError, match="suffix batch dim"):
        jag.add_suffix(torch.randn(3, 2, 4, device=DEV))
    short = JaggedTokens(tokens=torch.randn(1, 6, 4, device=DEV), weight=torch.ones(6, device=DEV),
                         offset=torch.tensor([0, 1, 6], device=DEV))
    with pytest.raises(ValueError, match="exceeds the length"):
        short.split_suffix(2)
    with pytest.raises(ValueError, match="Cannot strip"):
        JaggedTokens(tokens=torch.randn(1, 4, 4, device=DEV), weight=torch.ones(4, device=DEV),
                     offset=torch.tensor([0, 2, 4], device=DEV)).split_suffix(100)
