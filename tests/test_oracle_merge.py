"""The merge / split oracle against the reference's known-answer vectors, a
loop brute force and layout invariants (CPU only)."""

import numpy as np
import pytest
import torch

import oracle
from bruteforce import merge_1d_loops, merge_2d_loops
from golden_cases import MERGE_1D, MERGE_2D


@pytest.mark.parametrize("case", MERGE_1D, ids=[c["name"] for c in MERGE_1D])
def test_golden_1d(case):
    jag, rev = oracle.token_merge_1d(case["tokens"], case["start_index"], case["group_size"], case["mask"])
    torch.testing.assert_close(jag.tokens, case["out"])
    assert torch.equal(jag.offset, case["offset"])
    assert torch.equal(rev, case["rev"])
    torch.testing.assert_close(jag.weight, case["weight"], rtol=0, atol=0)
    B, N, C = case["tokens"].shape
    torch.testing.assert_close(oracle.token_split(jag, rev, (1, B, N, C)), case["restore"])


@pytest.mark.parametrize("case", MERGE_2D, ids=[c["name"] for c in MERGE_2D])
def test_golden_2d(case):
    jag, rev = oracle.token_merge_2d(
        case["tokens"], case["start_index"], case["group_h"], case["group_w"], case["H"], case["W"], case["mask"]
    )
    torch.testing.assert_close(jag.tokens, case["out"])
    assert torch.equal(jag.offset, case["offset"])
    assert torch.equal(rev, case["rev"])
    torch.testing.assert_close(jag.weight, case["weight"], rtol=0, atol=0)
    B, N, C = case["tokens"].shape
    torch.testing.assert_close(oracle.token_split(jag, rev, (1, B, N, C)), case["restore"])


@pytest.mark.parametrize("B,M,G,S,C,tail", [(1, 4, 2, 0, 3, 0), (3, 5, 3, 2, 4, 0), (2, 7, 9, 5, 2, 0),
                                            (2, 3, 4, 1, 5, 3), (2, 0, 4, 3, 2, 0), (1, 6, 1, 0, 2, 2)])
def test_bruteforce_1d(B, M, G, S, C, tail):
    N = S + M * G + tail
    tokens = torch.randn(B, N, C, dtype=torch.float64)
    mask = torch.rand(B, M) < 0.5
    jag, rev = oracle.token_merge_1d(tokens, S, G, mask, tail=tail)
    out, offset, rev_bf, weight = merge_1d_loops(tokens.numpy(), S, G, mask.numpy(), tail)
    np.testing.assert_allclose(jag.tokens[0].numpy(), out, rtol=1e-12, atol=1e-12)
    assert jag.offset.tolist() == offset.tolist()
    assert rev.tolist() == rev_bf.tolist()
    assert jag.weight.tolist() == weight.tolist()


@pytest.mark.parametrize("B,H,W,gh,gw,S,C", [(1, 4, 4, 2, 2, 0, 2), (2, 4, 6, 2, 3, 1, 3), (2, 7, 7, 3, 3, 2, 2),
                                             (1, 5, 8, 2, 3, 0, 1), (2, 37, 37, 3, 3, 5, 1), (1, 2, 2, 3, 3, 1, 2)])
def test_bruteforce_2d_incl_remainder(B, H, W, gh, gw, S, C):
    N = S + H * W
    M = (H // gh) * (W // gw)
    tokens = torch.randn(B, N, C, dtype=torch.float64)
    mask = torch.rand(B, M) < 0.5
    jag, rev = oracle.token_merge_2d(tokens, S, gh, gw, H, W, mask, allow_remainder=True)
    out, offset, rev_bf, weight = merge_2d_loops(tokens.numpy(), S, gh, gw, H, W, mask.numpy())
    np.testing.assert_allclose(jag.tokens[0].numpy(), out, rtol=1e-12, atol=1e-12)
    assert jag.offset.tolist() == offset.tolist()
    assert rev.tolist() == rev_bf.tolist()
    assert jag.weight.tolist() == weight.tolist()


def test_remainder_flag_is_noop_on_divisible_grid():
    tokens = torch.randn(2, 1 + 6 * 9, 4)
    mask = torch.rand(2, 6) < 0.5
    a, ra = oracle.token_merge_2d(tokens, 1, 3, 3, 6, 9, mask)
    b, rb = oracle.token_merge_2d(tokens, 1, 3, 3, 6, 9, mask, allow_remainder=True)
    assert torch.equal(a.tokens, b.tokens) and torch.equal(ra, rb) and torch.equal(a.offset, b.offset)


def test_invariants_large():
    B, M, G, S, C = 4, 64, 9, 5, 8
    N = S + M * G
    tokens = torch.randn(B, N, C)
    mask = torch.rand(B, M) < 0.4
    jag, rev = oracle.token_merge_1d(tokens, S, G, mask)
    P = jag.tokens.shape[1]
    k = int(mask.sum())
    assert P == B * N - k * (G - 1) == int(jag.offset[-1])
    assert float(jag.weight.sum()) == B * N
    assert set(rev.tolist()) == set(range(P))                       # onto
    r = rev.reshape(B, N)
    assert bool((r[:, 1:] >= r[:, :-1]).all())                      # monotone inside a frame (1-D)
    restored = oracle.token_split(jag, rev, (1, B, N, C))
    grouped = tokens[:, S:].reshape(B, M, G, C)
    want = torch.where(mask[:, :, None, None], grouped.mean(2, keepdim=True).expand_as(grouped), grouped)
    torch.testing.assert_close(restored[:, S:].reshape(B, M, G, C), want)
    assert torch.equal(restored[:, :S], tokens[:, :S])


@pytest.mark.parametrize("value", [True, False])
def test_uniform_masks(value):
    B, M, G, S, C = 2, 8, 4, 2, 3
    tokens = torch.randn(B, S + M * G, C)
    mask = torch.full((B, M), value)
    jag, rev = oracle.token_merge_1d(tokens, S, G, mask)
    if value:
        want = torch.cat([tokens[:, :S], tokens[:, S:].reshape(B, M, G, C).mean(2)], dim=1).reshape(1, -1, C)
        torch.testing.assert_close(jag.tokens, want)
    else:
        assert torch.equal(jag.tokens, tokens.reshape(1, -1, C))
        assert rev.tolist() == list(range(B * (S + M * G)))


def test_bf16_mean_is_fp32_accumulate_single_rounding():
    # nine tokens of 33.0: a bf16 running sum gives 296/9 -> 32.875, the oracle must give 33.0
    tokens = torch.full((1, 9, 2), 33.0, dtype=torch.bfloat16)
    jag, _ = oracle.token_merge_1d(tokens, 0, 9, torch.tensor([[True]]))
    assert jag.tokens.dtype == torch.bfloat16
    assert jag.tokens.float().tolist() == [[[33.0, 33.0]]]
    x = torch.randn(3, 9 * 7, 16).bfloat16()
    jag, _ = oracle.token_merge_1d(x, 0, 9, torch.ones(3, 7, dtype=torch.bool))
    want = x.float().reshape(3, 7, 9, 16).sum(2).div(9).bfloat16().reshape(1, 21, 16)
    assert torch.equal(jag.tokens, want)


@pytest.mark.parametrize("tokens,mask,start,G,msg", [
    (torch.randn(2, 7, 4), torch.ones(2, 3, dtype=torch.bool), 0, 2, "Expected N = start_index"),
    (torch.randn(2, 6, 4), torch.ones(3, 3, dtype=torch.bool), 0, 2, "merge_mask batch"),
    (torch.randn(1, 6, 4), torch.ones(1, 3, dtype=torch.bool), -1, 2, "start_index"),
    (torch.randn(1, 6, 4), torch.ones(1, 3, dtype=torch.bool), 0, 0, "group_size"),
    (torch.randn(1, 6, 4), torch.ones(1, 3, dtype=torch.float32), 0, 2, "torch.bool"),
])
def test_validation_1d(tokens, mask, start, G, msg):
    with pytest.raises(ValueError, match=msg):
        oracle.token_merge_1d(tokens, start, G, mask)


@pytest.mark.parametrize("tokens,mask,start,gh,gw,H,W,msg", [
    (torch.randn(1, 15, 4), torch.ones(1, 3, dtype=torch.bool), 0, 2, 3, 3, 5, "H.*divisible"),
    (torch.randn(1, 12, 4), torch.ones(1, 2, dtype=torch.bool), 0, 2, 5, 4, 3, "W.*divisible"),
    (torch.randn(2, 16, 4), torch.ones(3, 4, dtype=torch.bool), 0, 2, 2, 4, 4, "merge_mask batch"),
    (torch.randn(1, 10, 4), torch.ones(1, 4, dtype=torch.bool), 0, 2, 2, 4, 4, "Expected N"),
    (torch.randn(1, 16, 4), torch.ones(1, 2, dtype=torch.bool), 0, 2, 2, 4, 4, "Expected M"),
    (torch.randn(1, 16, 4), torch.ones(1, 4, dtype=torch.bool), -1, 2, 2, 4, 4, "start_index"),
    (torch.randn(1, 16, 4), torch.ones(1, 4, dtype=torch.bool), 0, 0, 2, 4, 4, "group_h.*group_w.*> 0"),
    (torch.randn(1, 16, 4), torch.ones(1, 4, dtype=torch.float32), 0, 2, 2, 4, 4, "torch.bool"),
])
def test_validation_2d(tokens, mask, start, gh, gw, H, W, msg):
    with pytest.raises(ValueError, match=msg):
        oracle.token_merge_2d(tokens, start, gh, gw, H, W, mask)
