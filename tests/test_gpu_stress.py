"""Long-sequence stress configuration on the GPU at full size: 128 frames of 37x28 patches + 5 special
tokens (133 248 tokens), 3x3 merge at ratio 0.75 with a per-frame jitter of +-0.1, so frame segments vary
between about 300 and 480 packed tokens and the global segment holds about 50 000.  The oracle cannot run
at this size in seconds, so the checks are size-independent properties and sampled rows / segments."""

import pytest
import torch

import oracle
from come_amd.cuda_extension import flash_attn_varlen_qkvpacked_func_w_perkey_bias
from come_amd.token_merger import func_token_merge, func_token_merge_2d, func_token_split

pytestmark = pytest.mark.gpu
DEV = "cuda"
FRAMES, H, W, S0 = 128, 37, 28, 5
N = S0 + H * W
M = (H // 3) * (W // 3)


def jittered_masks(seed):
    g = torch.Generator().manual_seed(seed)
    conf = torch.rand(FRAMES, M, generator=g)
    k = ((0.75 + (torch.rand(FRAMES, generator=g) * 2 - 1) * 0.1) * M).round().long()
    rank = conf.argsort(dim=1).argsort(dim=1)
    return rank < k[:, None], k


def test_merge_and_unmerge_properties():
    C = 1024
    mask, k = jittered_masks(0)
    g = torch.Generator().manual_seed(1)
    tokens = torch.randn(FRAMES, N, C, generator=g).bfloat16().to(DEV)
    jag, rev = func_token_merge_2d(tokens.view(FRAMES, N, C), S0, 3, 3, H, W, mask.to(DEV), allow_remainder=True)
    # offsets, bit-exact against the closed form: every merged window removes 8 rows of its frame
    lens = N - 8 * k
    want_offset = torch.cat((torch.zeros(1, dtype=torch.long), lens.cumsum(0)))
    assert torch.equal(jag.offset.cpu(), want_offset)
    P = int(want_offset[-1])
    assert jag.tokens.shape == (1, P, C)
    assert float(jag.weight.sum()) == FRAMES * N
    assert int((jag.weight == 9).sum()) == int(k.sum()) and int((jag.weight == 1).sum()) == P - int(k.sum())
    # the index map is onto, and stays inside the frame's segment
    assert int(torch.bincount(rev, minlength=P).min()) >= 1
    seg = torch.bucketize(rev.cpu(), want_offset[1:], right=True)
    assert torch.equal(seg, torch.arange(FRAMES).repeat_interleave(N))
    # unmerge: kept tokens come back bit-exact, merged ones as the mean of their window
    restored = func_token_split(jag, rev, (1, FRAMES, N, C)).reshape(FRAMES, N, C)
    kept = (jag.weight[rev] == 1).reshape(FRAMES, N)
    assert torch.equal(restored[kept], tokens[kept])
    grid = tokens[:, S0:].reshape(FRAMES, H, W, C)[:, :36, :27].reshape(FRAMES, 12, 3, 9, 3, C)
    means = grid.float().mean(dim=(2, 4)).bfloat16()                                     # [F, 12, 9, C]
    back = restored[:, S0:].reshape(FRAMES, H, W, C)[:, :36, :27].reshape(FRAMES, 12, 3, 9, 3, C)
    m = mask.reshape(FRAMES, 12, 9).to(DEV)
    got = back[:, :, 0, :, 0][m].float()
    # one rounding of an fp32 mean on both sides; the summation order may differ by one bf16 ulp
    torch.testing.assert_close(got, means[m].float(), rtol=2 ** -7, atol=1e-2)
    assert torch.equal(back[:, :, 1, :, 2][m], back[:, :, 0, :, 0][m])                     # whole window shares the row


def test_frame_and_global_attention_sampled():
    Hh, D = 16, 64
    mask, k = jittered_masks(2)
    lens = (N - 8 * k).tolist()
    assert 290 <= min(lens) and max(lens) <= 500
    P = sum(lens)
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(P, 3, Hh, D, generator=g).bfloat16()
    count = torch.ones(P)
    count[torch.randperm(P, generator=g)[: int(k.sum())]] = 9.0
    bias = count.log().bfloat16()
    bounds = [0]
    for n in lens:
        bounds.append(bounds[-1] + n)
    # frame mode: 128 segments; the first, the shortest, the longest and the last are checked in full
    cu = torch.tensor(bounds, dtype=torch.int32)
    out = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), max(lens), perkey_bias=bias.to(DEV),
                                                         softmax_scale=0.125).float().cpu()
    assert bool(torch.isfinite(out).all())
    for f in {0, lens.index(min(lens)), lens.index(max(lens)), FRAMES - 1}:
        s, e = bounds[f], bounds[f + 1]
        ref, _ = oracle.biased_varlen_attention(qkv[s:e], torch.tensor([0, e - s]), bias[s:e], 0.125)
        diff = (out[s:e] - ref).abs()
        assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
    # global mode: one segment of about 50 000 tokens; sampled rows against the closed form
    cu1 = torch.tensor([0, P], dtype=torch.int32)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu1.to(DEV), P, perkey_bias=bias.to(DEV),
                                                                 softmax_scale=0.125, return_attn_probs=True)
    out, lse = out.float().cpu(), lse.cpu()
    q, kk, v = qkv.float().unbind(1)
    for row in [0, 63, 64, 255, 256, 25000, P - 257, P - 1]:
        scores = torch.einsum("hd,khd->hk", q[row], kk) * 0.125 + bias.float()[None]
        ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v)
        diff = (out[row] - ref).abs()
        assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
        torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=2e-3, rtol=1e-3)


def test_unmerged_global_segment_of_133k_tokens_sampled():
    """The unmerged stress sequence as one segment (133 248 tokens, row stride 768 B -> 102 MB of packed q/k/v):
    exercises the large offsets; sampled rows against the closed form (2 heads keep it at 9 TFLOP)."""
    Hh, D, L = 2, 64, FRAMES * N
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(L, 3, Hh, D, generator=g).bfloat16()
    bias = (torch.rand(L, generator=g) * 2).bfloat16()
    cu = torch.tensor([0, L], dtype=torch.int32)
    out, lse, _ = flash_attn_varlen_qkvpacked_func_w_perkey_bias(qkv.to(DEV), cu.to(DEV), L, perkey_bias=bias.to(DEV),
                                                                 softmax_scale=0.125, return_attn_probs=True)
    out, lse = out.float().cpu(), lse.cpu()
    assert bool(torch.isfinite(out).all())
    q, k, v = qkv.float().unbind(1)
    for row in [0, 255, 256, 511, 512, 70000, L - 513, L - 1]:
        scores = torch.einsum("hd,khd->hk", q[row], k) * 0.125 + bias.float()[None]
        ref = torch.einsum("hk,khd->hd", torch.softmax(scores, -1), v)
        diff = (out[row] - ref).abs()
        assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3
        torch.testing.assert_close(lse[:, row], torch.logsumexp(scores, -1), atol=2e-3, rtol=1e-3)


def _needs_free_memory(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip(f"needs {gib} GiB of free device memory")


def test_unmerge_beyond_one_launch():
    """More than 2^31 (row, 16-byte chunk) items: the entry point covers the output with several launches over
    consecutive row ranges.  2.2 M rows of 16 KiB (36 GB) gathered from 1000 packed rows; rows around the launch
    border and at both ends are compared with the gather they stand for."""
    _needs_free_memory(60)
    from come_amd.cuda_extension import co_me_cuext
    C, P, total = 8192, 1000, 2_200_000
    assert total * (C * 2 // 16) > 2 ** 31
    g = torch.Generator(device=DEV).manual_seed(0)
    merged = torch.randn(P, C, device=DEV, generator=g).bfloat16()
    rev = torch.randint(0, P, (total,), device=DEV, generator=g, dtype=torch.int32)
    out = co_me_cuext.co_me_token_split_cuda(merged, rev, C)
    assert out.shape == (total, C)
    border = ((2 ** 31 - 1) // (C * 2 // 16)) // 256 * 256                      # first row of the second launch
    rows = torch.tensor([0, 1, 255, 256, border - 1, border, border + 1, border + 255, total - 2, total - 1], device=DEV)
    assert torch.equal(out[rows], merged[rev[rows].long()])
    step = torch.arange(0, total, 9973, device=DEV)
    assert torch.equal(out[step], merged[rev[step].long()])


def test_merge_beyond_one_launch():
    """The same for the merge: 4200 rows of 1032 tokens x 8192 channels (71 GB of bf16 tokens, 1-D groups of 2)
    exceed 2^31 (unit, chunk) items, so the rows are covered by two launches.  Frames at the ends and on both sides
    of the launch border are compared with the oracle."""
    _needs_free_memory(160)
    rows, S, M, G, C = 4200, 8, 512, 2, 8192
    N = S + M * G
    per_row_items = max(M, S) * (C * 2 // 16)
    border = (2 ** 31 - 1) // per_row_items                                          # first row of the second launch
    assert 0 < border < rows
    # small integers: every mean of two of them is exact in bf16, so packed rows can be compared bit for bit
    pattern = (torch.arange(rows * N, device=DEV) % 61).to(torch.bfloat16).view(rows, N, 1)
    tokens = torch.empty(rows, N, C, dtype=torch.bfloat16, device=DEV)
    tokens.copy_(pattern)
    g = torch.Generator(device=DEV).manual_seed(1)
    mask = torch.rand(rows, M, device=DEV, generator=g) < 0.5
    jag, rev = func_token_merge(tokens, S, G, mask)
    P = jag.tokens.shape[1]
    assert P == rows * N - int(mask.sum()) * (G - 1) == int(jag.offset[-1])
    assert float(jag.weight.sum()) == rows * N
    for f in (0, border - 1, border, border + 1, rows - 1):
        ref, ref_rev = oracle.token_merge_1d(tokens[f:f + 1, :, :16].cpu(), S, G, mask[f:f + 1].cpu())
        lo, hi = int(jag.offset[f]), int(jag.offset[f + 1])
        assert hi - lo == ref.tokens.shape[1]
        got = jag.tokens[0, lo:hi]
        assert torch.equal(got[:, :16].cpu(), ref.tokens[0])
        assert torch.equal(got[:, -1].cpu(), ref.tokens[0][:, 0])                    # last channel chunk as well
        assert torch.equal(rev[f * N:(f + 1) * N].cpu() - lo, ref_rev)
        assert torch.equal(jag.weight[lo:hi].cpu(), ref.weight)
    del tokens
    back = func_token_split(jag, rev, (1, rows, N, C))
    idx = torch.tensor([0, N - 1, border * N - 1, border * N, rows * N - 1], device=DEV)
    assert torch.equal(back.view(-1, C)[idx], jag.tokens[0][rev[idx]])
