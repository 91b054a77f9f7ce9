"""Host-side argument checks of the drop-in Python layer (CPU only): the messages are the ones
the reference's tests match (test_token_merge_func.py:298-318, test_token_merge_2d.py:288-321)."""

import pytest
import torch

from come_amd.token_merger import func_token_merge, func_token_merge_2d
from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias


@pytest.mark.parametrize("tokens,mask,start,G,msg", [
    (torch.randn(2, 7, 4), torch.ones(2, 3, dtype=torch.bool), 0, 2, "Expected N = start_index"),
    (torch.randn(2, 6, 4), torch.ones(3, 3, dtype=torch.bool), 0, 2, "merge_mask batch"),
    (torch.randn(1, 6, 4), torch.ones(1, 3, dtype=torch.bool), -1, 2, "start_index"),
    (torch.randn(1, 6, 4), torch.ones(1, 3, dtype=torch.bool), 0, 0, "group_size"),
    (torch.randn(1, 6, 4), torch.ones(1, 3, dtype=torch.float32), 0, 2, "torch.bool"),
])
def test_merge_1d_validation(tokens, mask, start, G, msg):
    with pytest.raises(ValueError, match=msg):
        func_token_merge(tokens=tokens, merge_mask=mask, start_index=start, group_size=G)


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
def test_merge_2d_validation(tokens, mask, start, gh, gw, H, W, msg):
    with pytest.raises(ValueError, match=msg):
        func_token_merge_2d(tokens=tokens, merge_mask=mask, start_index=start, group_h=gh, group_w=gw, H=H, W=W)


def test_operators_refuse_cpu_tensors():
    # valid arguments on the CPU must not silently run somewhere else
    with pytest.raises(RuntimeError, match="CUDA"):
        func_token_merge(torch.randn(1, 6, 4), 0, 2, torch.ones(1, 3, dtype=torch.bool))
    qkv = torch.randn(8, 3, 2, 64).bfloat16()
    cu = torch.tensor([0, 8], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA"):
        flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, 8, perkey_bias=torch.zeros(8).bfloat16())


def test_split_pair_and_legacy_entry_points_on_the_host():
    from come_amd.cuda_extension import co_me_cuext
    a = torch.randn(4, 8)
    with pytest.raises(RuntimeError, match="CUDA"):
        co_me_cuext.co_me_token_split_pair_cuda(a, a, torch.zeros(3, dtype=torch.int64), 8)
    # the reference exports a first-generation pair that nothing calls (co_me_cuext.pyi:22-46): refused by name
    with pytest.raises(RuntimeError, match="not provided"):
        co_me_cuext.co_me_token_merge_cuda_legacy(0, a, a, None)
    with pytest.raises(RuntimeError, match="not provided"):
        co_me_cuext.co_me_token_merge_scan_legacy(0, 2, a)


def test_predictor_adapter_calls_reference_style_modules_with_the_shape():
    """The reference's predictor modules take ``BPHWC`` beside the tokens and return ``[B*S, H*W, 1]``
    (confidence_predictor.py:21-29, 51-75); a plain callable gets the tokens only."""
    from come_amd.token_merger.co_me import run_predictor

    class ReferenceStyle(torch.nn.Module):
        def forward(self, tokens, BPHWC):
            B, P, H, W, C = BPHWC
            assert tokens.shape == (B, P, H, W, C) and tokens.dtype == torch.bfloat16
            return tokens.reshape(B * P, H * W, C).float().mean(-1, keepdim=True)

    feature = torch.randn(2, 3, 8, 4, 5)                       # [B, S, C, H, W]
    want = feature.bfloat16().float().mean(2).reshape(6, 20)
    got = run_predictor(ReferenceStyle(), feature)
    assert got.shape == (6, 20, 1)
    torch.testing.assert_close(got.squeeze(-1), want, atol=1e-2, rtol=1e-2)
    plain = run_predictor(lambda t: t.float().mean(-1), feature)
    torch.testing.assert_close(plain.reshape(6, 20), want, atol=1e-2, rtol=1e-2)
    with pytest.raises(ValueError, match="one confidence per patch"):
        run_predictor(lambda t: t.float(), feature)


def test_scale_mode_choice_follows_the_bound_attached_by_the_prologue():
    """Host logic only: the norm bound of a LayerNorm'd head from its gain and bias, and the decision the attention
    operators derive from a tensor's ``come_qk_bound`` (no bound: never folded)."""
    from come_amd.common.qkv import _norm_bound
    from come_amd.cuda_extension.flash_attn import FOLD_SCALE_MAX_LOGIT, _fold_scale

    ln = torch.nn.LayerNorm(64)
    assert _norm_bound(ln.weight, ln.bias, 64, torch.bfloat16) == pytest.approx(8.0)
    with torch.no_grad():
        ln.weight.fill_(0.5)
        ln.weight[3] = -2.0
        ln.bias.fill_(0.25)
    assert _norm_bound(ln.weight, ln.bias, 64, torch.bfloat16) == pytest.approx(8.0 * 2.0 + 0.25 * 8.0)   # new version, new value
    assert _norm_bound(None, None, 64, torch.float16) == pytest.approx(8.0)
    # the bound really bounds the norm of any normalised head
    x = torch.randn(1000, 64) * 5 + 3
    y = torch.nn.functional.layer_norm(x, (64,), ln.weight.detach(), ln.bias.detach())
    assert float(y.norm(dim=-1).max()) <= _norm_bound(ln.weight, ln.bias, 64, torch.float32)

    t = torch.zeros(4, 3, 2, 64)
    assert _fold_scale(t, 0.125, "auto") is False
    assert _fold_scale(t, 0.125, "folded") is True and _fold_scale(t, 0.125, "exact") is False
    t.come_qk_bound = FOLD_SCALE_MAX_LOGIT / 0.125
    assert _fold_scale(t, 0.125, "auto") is True
    t.come_qk_bound = FOLD_SCALE_MAX_LOGIT / 0.125 * 1.01
    assert _fold_scale(t, 0.125, "auto") is False
    with pytest.raises(ValueError, match="scale_mode"):
        _fold_scale(t, 0.125, "fast")
