"""Pins for the biased varlen attention oracle: loop brute force, reductions
to torch SDPA, the key-duplication identity behind log(count), logsumexp."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from bruteforce import attention_loops

SEGMENT_SETS = [[32, 48, 24, 24], [56, 49, 23], [128], [60, 40], [50], [128, 256], [100, 150, 50], [64] * 4]


def _cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


def test_vs_loops_tiny():
    lens, H, D = [5, 1, 7], 2, 4
    P = sum(lens)
    qkv = torch.randn(P, 3, H, D, dtype=torch.float64)
    bias = torch.randn(P, dtype=torch.float64)
    out, lse = oracle.biased_varlen_attention(qkv.float(), _cu(lens), bias.float(), softmax_scale=0.3)
    cu = _cu(lens).tolist()
    for s, e in zip(cu[:-1], cu[1:]):
        for h in range(H):
            o, l = attention_loops(qkv[s:e, 0, h].numpy(), qkv[s:e, 1, h].numpy(), qkv[s:e, 2, h].numpy(),
                                   bias[s:e].numpy(), 0.3)
            np.testing.assert_allclose(out[s:e, h].numpy(), o, rtol=2e-5, atol=2e-6)
            np.testing.assert_allclose(lse[h, s:e].numpy(), l, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("lens", SEGMENT_SETS)
def test_vs_reference_test_closed_form(lens):
    # the formula the reference's tests use, per segment and head (test_flex_attention_bias.py:26-36)
    H, D = 4, 64
    P = sum(lens)
    qkv = torch.randn(P, 3, H, D).bfloat16()
    weight = torch.rand(P).clamp(min=1e-3)
    bias = weight.log().bfloat16()
    out, _ = oracle.biased_varlen_attention(qkv, _cu(lens), bias)
    q, k, v = qkv.float().unbind(1)
    cu = _cu(lens).tolist()
    for s, e in zip(cu[:-1], cu[1:]):
        for h in range(H):
            a = torch.softmax((q[s:e, h] @ k[s:e, h].T) * (D ** -0.5) + bias.float()[None, s:e], dim=-1)
            torch.testing.assert_close(out[s:e, h], a @ v[s:e, h], rtol=1e-5, atol=1e-6)


def test_zero_bias_is_plain_sdpa_and_none():
    lens, H, D = [64, 37], 2, 64
    P = sum(lens)
    qkv = torch.randn(P, 3, H, D)
    a, la = oracle.biased_varlen_attention(qkv, _cu(lens), torch.zeros(P))
    b, lb = oracle.biased_varlen_attention(qkv, _cu(lens), None)
    assert torch.equal(a, b) and torch.equal(la, lb)
    cu = _cu(lens).tolist()
    for s, e in zip(cu[:-1], cu[1:]):
        q, k, v = (qkv[s:e, i].transpose(0, 1)[None] for i in range(3))
        ref = F.scaled_dot_product_attention(q, k, v)[0].transpose(0, 1)
        torch.testing.assert_close(a[s:e], ref, rtol=1e-5, atol=1e-6)


def test_count_equals_key_duplication():
    # a key with bias log(c) acts exactly like that key (and its value) repeated c times
    L, H, D, c = 9, 2, 8, 9
    qkv = torch.randn(L, 3, H, D, dtype=torch.float64).float()
    count = torch.ones(L)
    count[3] = c
    a, la = oracle.biased_varlen_attention(qkv, _cu([L]), count.log())
    dup = torch.cat([qkv, qkv[3:4].repeat(c - 1, 1, 1, 1)])
    b, lb = oracle.biased_varlen_attention(dup, _cu([L + c - 1]), None)
    torch.testing.assert_close(a, b[:L], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(la, lb[:, :L], rtol=1e-5, atol=1e-6)


def test_segments_are_isolated_and_permutable():
    lens, H, D = [10, 20, 7], 2, 16
    P = sum(lens)
    qkv, bias = torch.randn(P, 3, H, D), torch.randn(P)
    out, _ = oracle.biased_varlen_attention(qkv, _cu(lens), bias)
    order = torch.cat([torch.arange(30, 37), torch.arange(0, 10), torch.arange(10, 30)])
    out_p, _ = oracle.biased_varlen_attention(qkv[order], _cu([7, 10, 20]), bias[order])
    torch.testing.assert_close(out_p, out[order], rtol=1e-5, atol=1e-6)
    qkv2 = qkv.clone()
    qkv2[10:30] += 5.0                                             # touching segment 1 leaves 0 and 2 alone
    out2, _ = oracle.biased_varlen_attention(qkv2, _cu(lens), bias)
    assert torch.equal(out2[:10], out[:10]) and torch.equal(out2[30:], out[30:])


def test_chunking_is_transparent_and_empty_segment():
    lens, H, D = [0, 33, 0, 5], 1, 8
    P = sum(lens)
    qkv, bias = torch.randn(P, 3, H, D), torch.randn(P)
    a, la = oracle.biased_varlen_attention(qkv, _cu(lens), bias, q_chunk=7)
    b, lb = oracle.biased_varlen_attention(qkv, _cu(lens), bias, q_chunk=4096)
    torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(la, lb, rtol=1e-6, atol=1e-7)


def test_sdpa_bf16_baseline_close_to_fp32_oracle():
    lens, H, D = [70, 58], 4, 64
    P = sum(lens)
    qkv = torch.randn(P, 3, H, D).bfloat16()
    bias = torch.where(torch.rand(P) < 0.3, math.log(9.0), 0.0).bfloat16()
    a, _ = oracle.biased_varlen_attention(qkv, _cu(lens), bias)
    b = oracle.biased_varlen_attention_sdpa_bf16(qkv, _cu(lens), bias)
    assert float((a - b.float()).abs().max()) < 3e-2
