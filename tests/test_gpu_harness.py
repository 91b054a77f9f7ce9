"""End-to-end harness on the GPU: the HIP operators against the oracle operators inside the same
bf16 model (same weights, same GEMMs; only merge / unmerge / selection / attention differ), and the
merged model against the unmerged one."""

import pytest
import torch

from come_amd.harness import AggregatorConfig, AlternatingAggregator, relative_l1
from harness_oracle import OracleMerger, oracle_attention, oracle_prologue

pytestmark = pytest.mark.gpu


def build(dim, heads, depth, merge_block, taps, seed=0, layer_scale=0.01):
    torch.manual_seed(seed)
    cfg = AggregatorConfig(dim=dim, heads=heads, mlp_dim=4 * dim, depth=depth, merge_block=merge_block, taps=taps,
                           head_hidden=64, conf_hidden=64, layer_scale=layer_scale)
    return AlternatingAggregator(cfg).eval().to(device="cuda", dtype=torch.bfloat16)


def hip_merger(ratio):
    from come_amd.token_merger import CoMe_2D_TokenMerger

    return CoMe_2D_TokenMerger(5, 3, 3, ratio, allow_remainder=True)


def test_kernel_path_matches_oracle_path():
    model = build(256, 4, 3, 1, (1, 2))
    images = torch.rand(1, 2, 3, 518, 518, generator=torch.Generator().manual_seed(3)).cuda()
    hip = model(images, merger=hip_merger(0.5))
    ref = model(images, merger=OracleMerger(5, 3, 3, 0.5), attention=oracle_attention, prologue=oracle_prologue)
    assert hip["tokens_packed"] == ref["tokens_packed"] == 1596
    assert torch.equal(hip["merge_mask"].cpu(), ref["merge_mask"])
    # stated tolerance for the kernel path against the oracle path of the same merged model
    assert relative_l1(hip["maps"], ref["maps"]) < 1e-2


def test_kernel_path_matches_oracle_path_where_attention_errors_would_show():
    """The full block width (dim 1024, 16 heads of 64), LayerScale 1.0 - every attention output enters the residual
    stream undamped - and q / k-norm gains drawn from U(0.5, 2) with small biases, as trained layers have them (logits
    of tens of nats): a wrong choice of attention arithmetic or a kernel error of a few per cent shows in the output
    maps here.  Same weights and GEMMs on both sides; merge, selection, prologue and attention differ."""
    # merging from block 0 on: the confidence comes from the embeddings, so both paths select from identical numbers
    model = build(1024, 16, 3, 0, (1, 2), layer_scale=1.0)
    g = torch.Generator().manual_seed(11)
    with torch.no_grad():
        for blk in list(model.frame_blocks) + list(model.global_blocks):
            for norm in (blk.q_norm, blk.k_norm):
                norm.weight.copy_((0.5 + 1.5 * torch.rand(64, generator=g)).to(norm.weight))
                norm.bias.copy_((0.1 * torch.randn(64, generator=g)).to(norm.bias))
    images = torch.rand(1, 2, 3, 518, 518, generator=torch.Generator().manual_seed(6)).cuda()
    hip = model(images, merger=hip_merger(0.5))
    ref = model(images, merger=OracleMerger(5, 3, 3, 0.5), attention=oracle_attention, prologue=oracle_prologue)
    assert hip["tokens_packed"] == ref["tokens_packed"]
    assert torch.equal(hip["merge_mask"].cpu(), ref["merge_mask"])
    assert bool(torch.isfinite(hip["maps"]).all())
    assert relative_l1(hip["maps"], ref["maps"]) < 1e-2


def test_unmerged_kernel_path_matches_oracle_path():
    model = build(256, 4, 2, 1, (0, 1))
    images = torch.rand(1, 2, 3, 518, 518, generator=torch.Generator().manual_seed(4)).cuda()
    hip = model(images, merger=None)
    ref = model(images, merger=None, attention=oracle_attention, prologue=oracle_prologue)
    assert relative_l1(hip["maps"], ref["maps"]) < 1e-2


def test_merged_close_to_unmerged():
    model = build(1024, 16, 4, 1, (1, 3))
    images = torch.rand(1, 4, 3, 518, 518, generator=torch.Generator().manual_seed(5)).cuda()
    dense = model(images, merger=None)
    merged = model(images, merger=hip_merger(0.5))
    assert merged["tokens_dense"] == 4 * 1374 and merged["tokens_packed"] == 4 * 78 + 288 + 288 * 9
    mask = merged["merge_mask"].reshape(4, 12, 12)
    keep = torch.ones(4, 37, 37, dtype=torch.bool, device="cuda")
    keep[:, :36, :36] = ~mask.repeat_interleave(3, 1).repeat_interleave(3, 2)
    keep_px = keep.repeat_interleave(14, 1).repeat_interleave(14, 2)[None, :, None]
    # stated end-to-end tolerance (random-init weights, bf16): relative L1 <= 5e-2 on pixels of unmerged windows
    assert relative_l1(merged["maps"], dense["maps"], keep_px) < 5e-2
    same = model(images, merger=hip_merger(0.0))
    assert same["tokens_packed"] == same["tokens_dense"]
    assert relative_l1(same["maps"], dense["maps"]) < 1e-2


def test_deferred_q_prologue_gives_the_same_bits_end_to_end():
    """The whole model with the q half of every attention prologue left to the attention kernel
    (``deferred_q_prologue``): merged and unmerged forward, the same output bits as with the in-place pass."""
    from come_amd.harness import deferred_q_prologue

    model = build(256, 4, 3, 1, (1, 2))
    images = torch.rand(1, 2, 3, 518, 518, generator=torch.Generator().manual_seed(5)).cuda()
    for merger in (hip_merger(0.5), None):
        two_step = model(images, merger=merger)
        fused = model(images, merger=merger, prologue=deferred_q_prologue)
        assert torch.equal(two_step["maps"], fused["maps"])
