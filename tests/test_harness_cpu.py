"""End-to-end harness on the CPU with the oracle operators (no GPU): the plumbing configuration
(2 frames of 518x518 -> 37x37 patches + 5 special tokens = 1374 tokens per frame, 4 frame + 4 global
blocks, fp32, lowest 50 % of the 3x3 windows merged)."""

import torch

from come_amd.harness import AggregatorConfig, AlternatingAggregator, relative_l1
from harness_oracle import OracleMerger, oracle_attention, oracle_prologue


def build(dim, heads, depth, merge_block, taps, seed=0):
    torch.manual_seed(seed)
    cfg = AggregatorConfig(dim=dim, heads=heads, mlp_dim=4 * dim, depth=depth, merge_block=merge_block, taps=taps,
                           head_hidden=64, conf_hidden=64)
    return AlternatingAggregator(cfg).eval()


def test_plumbing_configuration_token_counts():
    model = build(1024, 16, 4, 1, (1, 3))
    images = torch.rand(1, 2, 3, 518, 518, generator=torch.Generator().manual_seed(1))
    out = model(images, merger=OracleMerger(5, 3, 3, 0.5), attention=oracle_attention, prologue=oracle_prologue)
    assert out["grid"] == (37, 37)
    assert out["tokens_dense"] == 2 * 1374 == 2748
    assert out["tokens_packed"] == 1596          # 2*(5+73) + 144 merged + 144*9 kept
    assert out["maps"].shape == (1, 2, 4, 518, 518)
    assert torch.isfinite(out["maps"]).all()


def test_merged_close_to_unmerged_and_ratio_zero_is_identity():
    model = build(128, 2, 3, 1, (1, 2))
    images = torch.rand(1, 3, 3, 126, 98, generator=torch.Generator().manual_seed(2))     # 9x7 patch grid
    dense = model(images, merger=None, attention=oracle_attention, prologue=oracle_prologue)
    same = model(images, merger=OracleMerger(5, 3, 3, 0.0), attention=oracle_attention, prologue=oracle_prologue)
    assert same["tokens_packed"] == same["tokens_dense"]
    # ratio 0 only reorders the tokens of a frame (window-major): equal up to fp32 summation order
    assert relative_l1(same["maps"], dense["maps"]) < 1e-5
    merged = model(images, merger=OracleMerger(5, 3, 3, 0.5), attention=oracle_attention, prologue=oracle_prologue)
    assert merged["tokens_packed"] < merged["tokens_dense"]
    # stated end-to-end tolerance for random-init weights: relative L1 <= 5e-2 on the pixels of unmerged windows
    mask = merged["merge_mask"].reshape(3, 3, 2)                                            # [frames, 3, 2] windows
    keep = torch.ones(3, 9, 7, dtype=torch.bool)
    keep[:, :9, :6] = ~mask.repeat_interleave(3, 1).repeat_interleave(3, 2)
    keep_px = keep.repeat_interleave(14, 1).repeat_interleave(14, 2)[None, :, None]
    assert relative_l1(merged["maps"], dense["maps"], keep_px) < 5e-2
