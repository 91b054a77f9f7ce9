"""GPU parity: token merge / unmerge through the C-ABI library against the CPU oracle and
the reference's known-answer vectors.  Index maps, counts and offsets must be bit-exact."""

import pytest
import torch

import oracle
from come_amd.cuda_extension import co_me_cuext
from come_amd.token_merger import func_token_merge, func_token_merge_2d, func_token_split
from golden_cases import MERGE_1D, MERGE_2D

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _assert_features(got, want, dtype):
    got, want = got.float().cpu(), want.float()
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)       # test_token_merge_cuda.py:102
    else:
        diff = (got - want).abs()
        assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3   # stated bf16 tolerance


def _check_against_oracle(tokens, S, G, mask):
    ref, ref_rev = oracle.token_merge_1d(tokens, S, G, mask)
    jag, rev = func_token_merge(tokens.to(DEV), S, G, mask.to(DEV))
    assert jag.offset.dtype == torch.int64 and rev.dtype == torch.int64 and jag.weight.dtype == torch.float32
    assert torch.equal(jag.offset.cpu(), ref.offset)
    assert torch.equal(rev.cpu(), ref_rev)
    assert torch.equal(jag.weight.cpu(), ref.weight)
    _assert_features(jag.tokens, ref.tokens, tokens.dtype)
    B, N, C = tokens.shape
    restored = func_token_split(jag, rev, (1, B, N, C))
    assert torch.equal(restored.cpu(), jag.tokens[0].cpu()[ref_rev].reshape(B, N, C))   # a gather is bit-exact
    return jag, ref


@pytest.mark.parametrize("case", MERGE_1D, ids=[c["name"] for c in MERGE_1D])
def test_golden_1d(case):
    jag, rev = func_token_merge(case["tokens"].to(DEV), case["start_index"], case["group_size"], case["mask"].to(DEV))
    torch.testing.assert_close(jag.tokens.cpu(), case["out"])
    assert torch.equal(jag.offset.cpu(), case["offset"])
    assert torch.equal(rev.cpu(), case["rev"])
    assert torch.equal(jag.weight.cpu(), case["weight"])
    B, N, C = case["tokens"].shape
    torch.testing.assert_close(func_token_split(jag, rev, (1, B, N, C)).cpu(), case["restore"])


@pytest.mark.parametrize("case", MERGE_2D, ids=[c["name"] for c in MERGE_2D])
def test_golden_2d(case):
    jag, rev = func_token_merge_2d(case["tokens"].to(DEV), case["start_index"], case["group_h"], case["group_w"],
                                   case["H"], case["W"], case["mask"].to(DEV))
    torch.testing.assert_close(jag.tokens.cpu(), case["out"])
    assert torch.equal(jag.offset.cpu(), case["offset"])
    assert torch.equal(rev.cpu(), case["rev"])
    assert torch.equal(jag.weight.cpu(), case["weight"])
    B, N, C = case["tokens"].shape
    torch.testing.assert_close(func_token_split(jag, rev, (1, B, N, C)).cpu(), case["restore"])


# shapes of the reference's randomised test (test_token_merge_cuda.py:77-88) plus 3x3-sized groups
RANDOM_1D = [(1, 4, 2, 0, 8), (2, 8, 2, 1, 16), (4, 16, 4, 2, 32), (8, 32, 4, 0, 64), (2, 64, 8, 4, 128),
             (16, 128, 2, 0, 256), (1, 256, 4, 1, 512), (4, 512, 2, 0, 1024), (2, 1024, 4, 2, 512),
             (3, 144, 9, 5, 1024), (2, 100, 9, 5, 2), (2, 7, 3, 1, 5), (1, 70, 5, 0, 24)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("B,M,G,S,C", RANDOM_1D)
def test_random_1d_vs_oracle(B, M, G, S, C, dtype):
    tokens = torch.randn(B, S + M * G, C).to(dtype)
    ratio = float(torch.rand(1)) * 0.8 + 0.1
    mask = torch.rand(B, M) < ratio
    _check_against_oracle(tokens, S, G, mask)


@pytest.mark.parametrize("value", [True, False])
def test_uniform_masks(value):
    B, M, G, S, C = 4, 32, 4, 2, 64
    tokens = torch.randn(B, S + M * G, C)
    _check_against_oracle(tokens, S, G, torch.full((B, M), value))


def test_group_size_one_and_no_groups():
    tokens = torch.randn(2, 17, 32)
    _check_against_oracle(tokens, 1, 1, torch.rand(2, 16) < 0.5)
    tokens = torch.randn(3, 5, 16)                               # M == 0: only special tokens
    _check_against_oracle(tokens, 5, 4, torch.zeros(3, 0, dtype=torch.bool))


def test_bf16_mean_is_fp32_accumulate_single_rounding():
    tokens = torch.full((1, 9, 8), 33.0, dtype=torch.bfloat16)
    jag, _ = func_token_merge(tokens.to(DEV), 0, 9, torch.ones(1, 1, dtype=torch.bool, device=DEV))
    assert jag.tokens.float().cpu().unique().tolist() == [33.0]
    x = torch.randn(4, 5 + 144 * 9, 1024).bfloat16()
    mask = torch.rand(4, 144) < 0.5
    ref, _ = oracle.token_merge_1d(x, 5, 9, mask)
    jag, _ = func_token_merge(x.to(DEV), 5, 9, mask.to(DEV))
    assert torch.equal(jag.tokens.cpu(), ref.tokens)             # same fp32 sum order, one rounding


RANDOM_2D = [(1, 4, 4, 2, 2, 0, 8), (2, 4, 6, 2, 3, 1, 16), (4, 8, 8, 4, 4, 0, 32), (2, 6, 6, 2, 3, 2, 64),
             (8, 8, 16, 4, 4, 0, 128), (1, 16, 16, 4, 8, 1, 256), (4, 8, 12, 2, 4, 0, 64), (2, 12, 12, 4, 6, 3, 32),
             (2, 36, 36, 3, 3, 5, 1024), (3, 12, 9, 3, 3, 5, 2)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,W,gh,gw,S,C", RANDOM_2D)
def test_random_2d_vs_oracle(B, H, W, gh, gw, S, C, dtype):
    tokens = torch.randn(B, S + H * W, C).to(dtype)
    mask = torch.rand(B, (H // gh) * (W // gw)) < 0.5
    ref, ref_rev = oracle.token_merge_2d(tokens, S, gh, gw, H, W, mask)
    jag, rev = func_token_merge_2d(tokens.to(DEV), S, gh, gw, H, W, mask.to(DEV))
    assert torch.equal(jag.offset.cpu(), ref.offset)
    assert torch.equal(rev.cpu(), ref_rev)
    assert torch.equal(jag.weight.cpu(), ref.weight)
    _assert_features(jag.tokens, ref.tokens, dtype)
    restored = func_token_split(jag, rev, (1, B, S + H * W, C))
    _assert_features(restored, oracle.token_split(ref, ref_rev, (1, B, S + H * W, C)), dtype)


@pytest.mark.parametrize("B,H,W,gh,gw,S,C", [(2, 37, 37, 3, 3, 5, 1024), (3, 37, 28, 3, 3, 5, 64), (2, 7, 7, 3, 3, 2, 2),
                                             (1, 5, 8, 2, 3, 0, 8), (2, 2, 2, 3, 3, 1, 8)])
def test_ragged_grid_remainder(B, H, W, gh, gw, S, C):
    tokens = torch.randn(B, S + H * W, C).bfloat16()
    mask = torch.rand(B, (H // gh) * (W // gw)) < 0.5
    ref, ref_rev = oracle.token_merge_2d(tokens, S, gh, gw, H, W, mask, allow_remainder=True)
    jag, rev = func_token_merge_2d(tokens.to(DEV), S, gh, gw, H, W, mask.to(DEV), allow_remainder=True)
    assert torch.equal(jag.offset.cpu(), ref.offset)
    assert torch.equal(rev.cpu(), ref_rev)
    assert torch.equal(jag.weight.cpu(), ref.weight)
    _assert_features(jag.tokens, ref.tokens, torch.bfloat16)
    with pytest.raises(ValueError, match="divisible"):
        func_token_merge_2d(tokens.to(DEV), S, gh, gw, H, W, mask.to(DEV))


def test_int32_index_map_and_counts_and_split():
    B, H, W, S, C = 4, 37, 37, 5, 256
    tokens = torch.randn(B, S + H * W, C).bfloat16()
    mask = torch.rand(B, 144) < 0.5
    ref, ref_rev = oracle.token_merge_2d(tokens, S, 3, 3, H, W, mask, allow_remainder=True)
    out, offsets, index_map, counts = co_me_cuext.co_me_token_merge_2d_cuda(
        tokens.to(DEV), S, 3, 3, H, W, mask.to(DEV), index_dtype=torch.int32, count_dtype=torch.int32)
    assert index_map.dtype == torch.int32 and counts.dtype == torch.int32 and offsets.dtype == torch.int32
    assert torch.equal(index_map.cpu().long(), ref_rev)
    assert torch.equal(counts.cpu().float(), ref.weight)
    assert torch.equal(offsets.cpu().long(), ref.offset)
    back = co_me_cuext.co_me_token_split_cuda(out, index_map, C)
    assert torch.equal(back.cpu(), out.cpu()[ref_rev])


def test_full_size_c2_properties():
    # merge microbenchmark shape: 16 frames of 37x37 (+5 specials), C = 1024, bf16
    B, H, W, S, C = 16, 37, 37, 5, 1024
    g = torch.Generator().manual_seed(0)
    tokens = torch.randn(B, S + H * W, C, generator=g).bfloat16().to(DEV)
    mask = (torch.rand(B, 144, generator=g) < 0.5).to(DEV)
    jag, rev = func_token_merge_2d(tokens, S, 3, 3, H, W, mask, allow_remainder=True)
    P = jag.tokens.shape[1]
    k = int(mask.sum())
    assert P == B * (S + H * W) - 8 * k == int(jag.offset[-1])
    assert float(jag.weight.sum()) == B * (S + H * W)
    assert int(rev.min()) == 0 and int(rev.max()) == P - 1
    assert int(torch.bincount(rev, minlength=P).min()) >= 1                     # onto
    restored = func_token_split(jag, rev, (1, B, S + H * W, C))
    kept = jag.weight[rev] == 1                                                   # unmerged tokens come back bit-exact
    assert torch.equal(restored.reshape(-1, C)[kept], tokens.reshape(-1, C)[kept])
    # merged tokens come back as their window mean: idempotent under a second merge + split
    jag2, rev2 = func_token_merge_2d(restored, S, 3, 3, H, W, mask, allow_remainder=True)
    assert torch.equal(rev2, rev)
    diff = (jag2.tokens.float() - jag.tokens.float()).abs()
    assert float(diff.max()) <= 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("C", [1024, 64, 12, 2, 1])
@pytest.mark.parametrize("index_dtype", [torch.int64, torch.int32], ids=["i64", "i32"])
def test_split_pair_is_two_splits_side_by_side(dtype, C, index_dtype):
    # the retained-layer step of the fused aggregator (reference vggt/fused.py:157-165): two token splits + cat
    P, total = 777, 2500
    g = torch.Generator().manual_seed(C)
    a = torch.randn(P, C, generator=g).to(dtype)
    b = torch.randn(P, C, generator=g).to(dtype)
    rev = torch.randint(0, P, (total,), generator=g)
    want = torch.cat((a[rev], b[rev]), dim=-1)                                    # a gather is bit-exact
    a_d, b_d, rev_d = a.to(DEV), b.to(DEV), rev.to(index_dtype).to(DEV)
    got = co_me_cuext.co_me_token_split_pair_cuda(a_d, b_d, rev_d, C)
    assert got.shape == (total, 2 * C) and got.dtype == dtype
    assert torch.equal(got.cpu(), want)
    assert torch.equal(got[:, :C], co_me_cuext.co_me_token_split_cuda(a_d, rev_d, C))
    assert torch.equal(got[:, C:], co_me_cuext.co_me_token_split_cuda(b_d, rev_d, C))


def test_split_pair_edges_and_errors():
    C = 256
    a = torch.randn(10, C).bfloat16().to(DEV)
    b = torch.randn(10, C).bfloat16().to(DEV)
    rev = torch.tensor([0, 9, -1, 10, 3], device=DEV)                              # out-of-range rows come back as zeros
    got = co_me_cuext.co_me_token_split_pair_cuda(a, b, rev, C).cpu()
    assert torch.equal(got[0], torch.cat((a[0], b[0])).cpu()) and torch.equal(got[4], torch.cat((a[3], b[3])).cpu())
    assert float(got[2].abs().max()) == 0 and float(got[3].abs().max()) == 0
    empty = co_me_cuext.co_me_token_split_pair_cuda(a, b, rev[:0], C)
    assert empty.shape == (0, 2 * C)
    no_rows = co_me_cuext.co_me_token_split_pair_cuda(a[:0], b[:0], rev, C)
    assert no_rows.shape == (5, 2 * C) and float(no_rows.abs().max()) == 0
    with pytest.raises(RuntimeError, match="merged_b must match"):
        co_me_cuext.co_me_token_split_pair_cuda(a, b[:5], rev, C)
    with pytest.raises(RuntimeError, match="merged_b must match"):
        co_me_cuext.co_me_token_split_pair_cuda(a, b.float(), rev, C)
    with pytest.raises(RuntimeError, match="rev_id must be"):
        co_me_cuext.co_me_token_split_pair_cuda(a, b, rev.float(), C)


@pytest.mark.parametrize("index_dtype", [torch.int64, torch.int32], ids=["i64", "i32"])
@pytest.mark.parametrize("dtype,C,total", [(torch.bfloat16, 512, 1001), (torch.bfloat16, 1024, 777), (torch.float32, 256, 333),
                                           (torch.bfloat16, 512, 70001), (torch.float32, 1024, 16401),
                                           (torch.float16, 1536, 21851)],
                         ids=["bf16-1seg", "bf16-2seg", "fp32-1seg", "bf16-two-rows-odd", "fp32-two-rows-odd", "fp16-3seg"])
def test_split_rows_of_whole_kibibytes(dtype, C, total, index_dtype):
    """Rows that are a multiple of 1 KiB wide take the wavefront-per-row kernel (one or two rows per wavefront
    depending on the launch size; an odd row count leaves a partial last group).  Indices outside the packed
    rows give rows of zeros."""
    P = 999
    g = torch.Generator().manual_seed(total)
    a = torch.randn(P, C, generator=g).to(dtype)
    b = torch.randn(P, C, generator=g).to(dtype)
    rev = torch.randint(0, P, (total,), generator=g)
    rev[[0, 5, total // 2, total - 1]] = torch.tensor([P - 1, -1, P, 0])
    rev[7] = 2 ** 40 if index_dtype == torch.int64 else 2 ** 31 - 1
    valid = (rev >= 0) & (rev < P)
    want_a = torch.where(valid[:, None], a[rev.clamp(0, P - 1)], torch.zeros((), dtype=dtype))
    want_b = torch.where(valid[:, None], b[rev.clamp(0, P - 1)], torch.zeros((), dtype=dtype))
    a_d, b_d, rev_d = a.to(DEV), b.to(DEV), rev.to(index_dtype).to(DEV)
    got = co_me_cuext.co_me_token_split_cuda(a_d, rev_d, C)
    assert torch.equal(got.cpu(), want_a)
    pair = co_me_cuext.co_me_token_split_pair_cuda(a_d, b_d, rev_d, C)
    assert torch.equal(pair.cpu(), torch.cat((want_a, want_b), dim=-1))


def test_split_pair_full_size_through_the_merger():
    from come_amd.token_merger import func_token_split_pair
    B, H, W, S, C = 16, 37, 37, 5, 1024
    g = torch.Generator().manual_seed(1)
    tokens = torch.randn(B, S + H * W, C, generator=g).bfloat16().to(DEV)
    mask = (torch.rand(B, 144, generator=g) < 0.5).to(DEV)
    jag, rev = func_token_merge_2d(tokens, S, 3, 3, H, W, mask, allow_remainder=True)
    other = type(jag)(tokens=jag.tokens.flip(1).contiguous(), weight=jag.weight, offset=jag.offset)
    shape = (1, B, S + H * W, C)
    both = func_token_split_pair(jag, other, rev, shape)
    assert both.shape == (B, S + H * W, 2 * C)
    assert torch.equal(both[..., :C], func_token_split(jag, rev, shape))
    assert torch.equal(both[..., C:], func_token_split(other, rev, shape))


def test_operators_run_on_the_current_stream():
    """The reference launches merge / split on the default stream whatever the caller's stream is
    (kernel_token_merge.cu:275); here every operator is enqueued on torch's current stream.  The inputs are
    produced on a side stream behind a few milliseconds of matrix products, so an operator that ran on another
    stream would read them before they exist."""
    from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias
    B, H, W, S, C = 4, 36, 36, 5, 256
    g = torch.Generator().manual_seed(3)
    tokens_cpu = torch.randn(B, S + H * W, C, generator=g).bfloat16()
    mask_cpu = torch.rand(B, 144, generator=g) < 0.5
    ref, ref_rev = oracle.token_merge_2d(tokens_cpu, S, 3, 3, H, W, mask_cpu)
    src, mask = tokens_cpu.to(DEV), mask_cpu.to(DEV)
    big = torch.randn(4096, 4096, device=DEV)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        acc = big
        for _ in range(20):
            acc = (acc @ big) * 1e-2                                    # a few milliseconds of work on the side stream
        tokens = torch.zeros_like(src)
        tokens += src + (acc[0, 0] * 0).to(src.dtype)                    # written behind the products, on the side stream
        jag, rev = func_token_merge_2d(tokens, S, 3, 3, H, W, mask)
        back = func_token_split(jag, rev, (1, B, S + H * W, C))
        qkv = jag.tokens[0, :, :192].reshape(-1, 3, 1, 64).contiguous()
        cu = jag.offset.to(torch.int32)
        out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv, cu, S + H * W, perkey_bias=jag.weight.log().bfloat16())
    side.synchronize()
    assert torch.equal(rev.cpu(), ref_rev) and torch.equal(jag.offset.cpu(), ref.offset)
    _assert_features(jag.tokens, ref.tokens, torch.bfloat16)
    assert torch.equal(back.cpu().reshape(-1, C), jag.tokens[0].cpu()[ref_rev])
    ref_out, _ = oracle.biased_varlen_attention(qkv.cpu(), cu.cpu(), jag.weight.log().bfloat16().cpu())
    diff = (out.float().cpu() - ref_out).abs()
    assert float(diff.max()) <= 1e-2
