"""Pins the oracle's rotary embedding by what the mathematics fixes (fp32, so rounding does not blur it)."""

import math

import torch

import oracle


def test_position_zero_is_identity():
    t = torch.randn(5, 3, 64)
    assert torch.equal(oracle.rope_2d(t, torch.zeros(5, 2, dtype=torch.long)), t)


def test_pairs_keep_their_norm_and_turn_by_the_closed_form_angle():
    t = torch.randn(7, 2, 64, dtype=torch.float64).float()
    pos = torch.tensor([[0, 3], [1, 0], [2, 5], [7, 7], [4, 1], [9, 2], [3, 3]])
    out = oracle.rope_2d(t, pos, base=100.0)
    for half, coord in ((0, 0), (1, 1)):                       # first half <- y, second half <- x
        for j in range(16):
            a, b = t[..., 32 * half + j], t[..., 32 * half + j + 16]
            oa, ob = out[..., 32 * half + j], out[..., 32 * half + j + 16]
            torch.testing.assert_close(oa * oa + ob * ob, a * a + b * b, rtol=1e-5, atol=1e-6)
            theta = pos[:, coord].float()[:, None] * (100.0 ** (-(2 * j) / 32))
            # counter-clockwise rotation of the pair (a, b) by theta
            torch.testing.assert_close(oa, a * theta.cos() - b * theta.sin(), rtol=1e-4, atol=1e-5)
            torch.testing.assert_close(ob, b * theta.cos() + a * theta.sin(), rtol=1e-4, atol=1e-5)


def test_scores_depend_on_relative_position_only():
    q, k = torch.randn(1, 1, 64), torch.randn(1, 1, 64)
    def score(pq, pk):
        rq = oracle.rope_2d(q, torch.tensor([pq]))
        rk = oracle.rope_2d(k, torch.tensor([pk]))
        return float((rq * rk).sum())
    assert math.isclose(score([5, 2], [3, 7]), score([9, 4], [7, 9]), rel_tol=1e-4, abs_tol=1e-4)
    assert not math.isclose(score([5, 2], [3, 7]), score([5, 2], [4, 7]), rel_tol=1e-3, abs_tol=1e-3)


def test_norm_then_rope_composition_and_v_untouched():
    torch.manual_seed(0)
    qkv = torch.randn(6, 3, 2, 64).bfloat16()
    w, b = torch.rand(64).bfloat16(), torch.randn(64).bfloat16()
    pos = torch.randint(0, 10, (6, 2))
    out = oracle.qk_norm_rope(qkv, w, b, w, b, 1e-5, pos)
    assert torch.equal(out[:, 2], qkv[:, 2])
    ln = torch.nn.functional.layer_norm(qkv[:, 0], (64,), w, b, 1e-5)
    assert torch.equal(out[:, 0], oracle.rope_2d(ln, pos))
    plain = oracle.qk_norm_rope(qkv, None, None, None, None, 1e-5, None)
    torch.testing.assert_close(plain[:, 1].float().mean(-1), torch.zeros(6, 2), atol=2e-2, rtol=0)
