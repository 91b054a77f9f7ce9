"""GPU parity: the 1-D merger class (groups of G consecutive tokens, the Pi3X configuration) in its three
confidence modes with several frames per batch element, against the oracle restatement of the reference's
``CoMe_TokenMerger.build_ctx`` (``src/accelerate/token_merger/co_me.py:47-73``), with merge / split /
build_infer_mask round trips."""

import pytest
import torch

import oracle
from come_amd.token_merger import CoMe_TokenMerger

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _exact_sum_confidence(B, S, HW, seed):
    """Values k / 2 with k in 0..30, arranged in pairs (v, 15 - v) inside every batch element: the mean is
    exactly 7.5 and every partial sum of values or of squared deviations is exact in fp32 in any order, so the
    long reductions of the normalised score cannot differ between implementations."""
    g = torch.Generator().manual_seed(seed)
    half = torch.randint(0, 31, (B, S * HW // 2), generator=g).float() / 2
    conf = torch.cat([half, 15.0 - half], dim=1)
    perm = torch.randperm(S * HW, generator=g)
    return conf[:, perm].contiguous()


@pytest.mark.parametrize("mode,threshold", [("pairwise-rank", 0.5), ("pairwise-rank", 0.3), ("abs_mse", 0.45),
                                            ("mse", -0.2), ("mse", 0.35)])
@pytest.mark.parametrize("B,S,H,W,G", [(2, 3, 4, 8, 4), (1, 4, 12, 12, 4), (3, 2, 6, 6, 9)])
def test_build_ctx_modes(B, S, H, W, G, mode, threshold):
    if mode == "mse":
        conf = _exact_sum_confidence(B, S, H * W, seed=B * 10 + S).bfloat16()
    else:
        conf = torch.rand(B, S * H * W, generator=torch.Generator().manual_seed(B * 10 + S)).bfloat16()
        conf[:, : H * W] += 1.0                                  # frame 0 differs: per-frame vs joint scope shows
    merger = CoMe_TokenMerger(start_idx=5, group_size=G, threshold=threshold, conf_mode=mode)
    feature = torch.empty(B, S, 8, H, W, device=DEV)
    mask, shape = merger.build_ctx(feature, confidence=conf.to(DEV))
    want = oracle.select_groups_1d(conf, B, S, G, threshold, mode=mode)
    assert shape == (B, S, 8, H, W)
    assert mask.shape == want.shape and mask.dtype == torch.bool
    assert torch.equal(mask.cpu(), want)
    assert 0 < int(want.sum()) < want.numel()
    if mode == "pairwise-rank":
        # per-frame quantile: frame 0, whose confidence is offset by +1, still merges its share; a joint quantile
        # over the batch element (the 2-D merger's scope) would merge nothing there
        joint = oracle.select_lowest_confidence(conf.reshape(B * S, 1, H * W), B, 1, G, threshold)
        assert int(joint[0].sum()) == 0 and not torch.equal(joint, want)
        if threshold == 0.5:
            assert int(want[0].sum()) > 0


def test_normalised_score_is_per_batch_element_not_per_frame():
    B, S, H, W, G = 2, 3, 4, 8, 4
    conf = _exact_sum_confidence(B, S, H * W, seed=5).bfloat16()
    merger = CoMe_TokenMerger(start_idx=0, group_size=G, threshold=-0.2, conf_mode="mse")
    mask, _ = merger.build_ctx(torch.empty(B, S, 8, H, W, device=DEV), confidence=conf.to(DEV))
    per_element = oracle.select_groups_1d(conf, B, S, G, -0.2, mode="mse")
    per_frame = oracle.select_groups_1d(conf.reshape(B * S, H * W), B * S, 1, G, -0.2, mode="mse")
    assert not torch.equal(per_element, per_frame)             # the data tells the two scopes apart
    assert torch.equal(mask.cpu(), per_element)


@pytest.mark.parametrize("mode,threshold", [("pairwise-rank", 0.5), ("abs_mse", 0.5), ("mse", 0.0)])
def test_merge_split_round_trip(mode, threshold):
    B, S, H, W, G, C, S0 = 2, 3, 8, 8, 4, 64, 5
    conf = (_exact_sum_confidence(B, S, H * W, seed=1) / 15).bfloat16()
    merger = CoMe_TokenMerger(start_idx=S0, group_size=G, threshold=threshold, conf_mode=mode)
    ctx = merger.build_ctx(torch.empty(B, S, C, H, W, device=DEV), confidence=conf.to(DEV))
    want_mask = oracle.select_groups_1d(conf, B, S, G, threshold, mode=mode)
    assert torch.equal(ctx[0].cpu(), want_mask)
    tokens = torch.randn(B, S, S0 + H * W, C).bfloat16()
    jag, stub = merger.merge(ctx, tokens.to(DEV))
    ref, ref_rev = oracle.token_merge_1d(tokens.flatten(0, 1), S0, G, want_mask)
    assert torch.equal(jag.offset.cpu(), ref.offset)
    assert torch.equal(stub[0].cpu(), ref_rev)
    assert torch.equal(jag.weight.cpu(), ref.weight)
    diff = (jag.tokens.float().cpu() - ref.tokens.float()).abs()
    assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
    back = merger.split(ctx, stub, jag)
    assert back.shape == tokens.shape
    assert torch.equal(back.cpu(), jag.tokens[0].cpu()[ref_rev].reshape(tokens.shape))
    infer = merger.build_infer_mask(ctx)
    assert infer.shape == (B, S, H, W) and infer.dtype == torch.bool
    assert torch.equal(infer.cpu().reshape(B * S, -1, G), want_mask[:, :, None].expand(-1, -1, G))
    kept = ~infer.reshape(B, S, H * W).cpu()
    assert torch.equal(back.cpu()[:, :, S0:][kept], tokens[:, :, S0:][kept])
    pair = merger.split_pair(ctx, stub, jag, jag)
    assert torch.equal(pair[..., :C], back) and torch.equal(pair[..., C:], back)
    # an explicit start_index overrides the merger's (reference co_me.py:89-91)
    jag0, stub0 = merger.merge(ctx, tokens[:, :, S0:].contiguous().to(DEV), start_index=0)
    ref0, ref0_rev = oracle.token_merge_1d(tokens[:, :, S0:].flatten(0, 1), 0, G, want_mask)
    assert torch.equal(jag0.offset.cpu(), ref0.offset) and torch.equal(stub0[0].cpu(), ref0_rev)


def test_validation():
    merger = CoMe_TokenMerger(start_idx=0, group_size=5, threshold=0.5)
    with pytest.raises(ValueError, match="divisible by group_size"):
        merger.build_ctx(torch.empty(1, 1, 4, 4, 4, device=DEV), confidence=torch.rand(1, 16, device=DEV))
    merger = CoMe_TokenMerger(start_idx=0, group_size=4, threshold=1.5)
    with pytest.raises(ValueError, match="threshold in"):
        merger.build_ctx(torch.empty(1, 1, 4, 4, 4, device=DEV), confidence=torch.rand(1, 16, device=DEV))
    merger = CoMe_TokenMerger(start_idx=0, group_size=4, threshold=0.5)
    with pytest.raises(ValueError, match="confidence tensor or a predictor"):
        merger.build_ctx(torch.empty(1, 1, 4, 4, 4, device=DEV))
