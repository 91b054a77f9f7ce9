"""GPU parity: window confidence means + lowest-confidence selection, and the fused
select + merge entry, against the CPU oracle.  Masks must be bit-exact."""

import pytest
import torch

import oracle
from come_amd.cuda_extension import co_me_cuext
from come_amd.token_merger import CoMe_2D_TokenMerger

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _smooth_confidence(frames, H, W, seed):
    """Beta(2,5) sample mixed 50/50 with a Gaussian-blurred (sigma 3, reflect) copy."""
    g = torch.Generator().manual_seed(seed)
    a = torch._standard_gamma(torch.full((frames, H, W), 2.0), generator=g)
    b = torch._standard_gamma(torch.full((frames, H, W), 5.0), generator=g)
    x = a / (a + b)
    r = min(9, H - 1, W - 1)
    ker = torch.exp(-torch.arange(-r, r + 1).float() ** 2 / (2 * 3.0 ** 2))
    ker = ker / ker.sum()
    y = torch.nn.functional.pad(x[:, None], (r, r, r, r), mode="reflect")
    y = torch.nn.functional.conv2d(y, ker.view(1, 1, 1, -1))
    y = torch.nn.functional.conv2d(y, ker.view(1, 1, -1, 1))[:, 0]
    return 0.5 * x + 0.5 * y


def _margin_ok(means, cut):
    return float((means - cut).abs().min()) >= 2.5e-7


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("batch,frames,H,W,ratio", [(1, 16, 37, 37, 0.25), (1, 16, 37, 37, 0.5), (1, 16, 37, 37, 0.75),
                                                    (2, 8, 36, 36, 0.5), (1, 32, 37, 37, 0.6), (3, 4, 12, 9, 0.37),
                                                    (1, 128, 37, 28, 0.75), (1, 2, 6, 6, 0.0), (1, 2, 6, 6, 1.0)])
def test_ranking_mask_bit_exact(batch, frames, H, W, ratio, dtype):
    conf = _smooth_confidence(batch * frames, H, W, seed=frames + H).to(dtype)
    want = oracle.select_lowest_confidence(conf, batch, 3, 3, ratio)
    mask, means = co_me_cuext.co_me_select_windows(conf.to(DEV), batch, 3, 3, ratio, return_means=True)
    ref_means = oracle.window_confidence_means(conf, 3, 3).float()
    if dtype == torch.bfloat16:
        assert torch.equal(means.cpu(), ref_means)
        assert torch.equal(mask.cpu(), want)
        return
    # fp32 confidence: torch's CPU sum of nine floats is not in index order (and depends on the build), so a
    # mean may differ from the oracle's in the last place.  Check the mean to that precision, and check the
    # selection itself bit-exactly by applying the reference's library calls to the very means the GPU made.
    torch.testing.assert_close(means.cpu(), ref_means, rtol=0, atol=1e-7)
    per_batch = means.cpu().reshape(batch, -1)
    cut = torch.quantile(per_batch, ratio, dim=-1, keepdim=True)
    assert torch.equal(mask.cpu(), (per_batch < cut).reshape(mask.shape))
    if torch.equal(means.cpu(), ref_means) or _margin_ok(ref_means.reshape(batch, -1), cut):
        assert torch.equal(mask.cpu(), want)


def test_ties_and_strictness():
    conf = torch.ones(4, 6, 6).bfloat16()
    mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, 0.5)
    assert int(mask.sum()) == 0                                    # all equal to the threshold: none merged
    conf[0] = 0.5
    mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, 0.5)
    assert torch.equal(mask.cpu(), oracle.select_lowest_confidence(conf, 1, 3, 3, 0.5))
    conf = (torch.randint(0, 4, (8, 12, 12)).float() / 4).bfloat16()   # heavy ties
    for ratio in (0.1, 0.3, 0.5, 0.9):
        mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 2, 3, 3, ratio)
        assert torch.equal(mask.cpu(), oracle.select_lowest_confidence(conf, 2, 3, 3, ratio))


def test_negative_values_and_absolute_mode():
    conf = torch.randn(6, 9, 9)
    mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, 0.4)
    assert torch.equal(mask.cpu(), oracle.select_lowest_confidence(conf, 1, 3, 3, 0.4))
    mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, 0.1, mode="abs_mse")
    assert torch.equal(mask.cpu(), oracle.select_lowest_confidence(conf, 1, 3, 3, 0.1, mode="abs_mse"))


def test_scalar_threshold_is_rounded_to_the_confidence_dtype():
    """`bf16 tensor < 0.45` compares against bf16(0.45) = 0.44921875: a window whose mean is exactly that value is
    not selected, although it is below 0.45 (reference co_me_2d.py:297-298 with a bf16 predictor output)."""
    conf = torch.full((2, 6, 6), 0.44921875).bfloat16()
    conf[1, :3, :3] = 0.4453125                                   # one step further down: selected
    for mode in ("abs_mse",):
        mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, 0.45, mode=mode)
        want = oracle.select_lowest_confidence(conf, 1, 3, 3, 0.45, mode=mode)
        assert want.reshape(-1).tolist() == [False] * 4 + [True] + [False] * 3
        assert torch.equal(mask.cpu(), want)
    # fp32 confidence keeps the fp32 threshold
    mask = co_me_cuext.co_me_select_windows(conf.float().to(DEV), 1, 3, 3, 0.45, mode="abs_mse")
    assert bool(mask.all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("batch,frames,H,W", [(1, 4, 12, 12), (2, 8, 37, 37), (1, 32, 37, 28)])
def test_normalised_score_mode(batch, frames, H, W, dtype):
    """z-score mode (not exercised by any test of the reference: parity unpinned there).  The mean and the
    standard deviation are long fp32 reductions whose last bit depends on the summation order, so the window
    means may differ from the CPU oracle's by a rounding step of the confidence dtype; the mask is compared
    bit for bit on every window whose oracle mean is further from the threshold than that, and those must be
    nearly all windows."""
    g = torch.Generator().manual_seed(batch * 100 + frames)
    conf = (torch.rand(batch * frames, H, W, generator=g) * 3 + 1).to(dtype)
    thr = -0.1
    mask, means = co_me_cuext.co_me_select_windows(conf.to(DEV), batch, 3, 3, thr, mode="mse", return_means=True)
    want = oracle.select_lowest_confidence(conf, batch, 3, 3, thr, mode="mse")
    flat = conf.reshape(batch, -1)
    z = (flat - flat.mean(dim=-1, keepdim=True)) / (flat.std(dim=-1, keepdim=True) + 1e-3)
    want_means = oracle.window_confidence_means(z.reshape(-1, H, W), 3, 3).float()
    step = 2.0 ** -6 if dtype == torch.bfloat16 else 1e-5
    torch.testing.assert_close(means.cpu(), want_means, atol=step, rtol=0)
    clear = (want_means - thr).abs() > step
    assert float(clear.float().mean()) > 0.9
    assert torch.equal(mask.cpu()[clear], want[clear])
    assert 0 < int(mask.sum()) < mask.numel()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_normalised_score_hand_computed_case(dtype):
    """Values 0, 1, 2, 3: mean 1.5, unbiased standard deviation sqrt(5 / 3) = 1.2909944, so
    z = (-1.5, -0.5, 0.5, 1.5) / 1.2919944 = (-1.1610, -0.3870, 0.3870, 1.1610) (bf16 rounds the denominator to
    1.2890625 and z to -1.1640625 ...).  The thresholds separate that from a biased deviation (z0 = -1.34) in
    both dtypes and, in fp32, from a missing + 1e-3 (z0 = -1.16190 instead of -1.16100)."""
    conf = torch.tensor([[[0.0, 1.0], [2.0, 3.0]]]).to(dtype)
    z = [-1.1609958, -0.3869986, 0.3869986, 1.1609958]
    thresholds = [-1.5, -1.25, -1.0, -0.5, -0.3, 0.0, 0.4, 1.0, 1.25]
    if dtype == torch.float32:
        thresholds += [-1.1615, -1.1605]
    for thr in thresholds:
        mask, means = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 1, 1, thr, mode="mse", return_means=True)
        assert mask.cpu().reshape(-1).tolist() == [v < thr for v in z], thr
        assert torch.equal(mask.cpu(), oracle.select_lowest_confidence(conf, 1, 1, 1, thr, mode="mse"))
        torch.testing.assert_close(means.cpu().reshape(-1), torch.tensor(z),
                                   atol=2.0 ** -8 if dtype == torch.bfloat16 else 2e-7, rtol=0)


def test_normalised_score_exact_sums_bit_exact():
    """Confidence whose sums are exact in fp32 in any order (half-integers in pairs v, 15 - v): the long
    reductions cannot depend on the summation order, so in bf16 the whole chain of rounded tensor operations
    must reproduce the oracle's mask and window means bit for bit."""
    g = torch.Generator().manual_seed(11)
    batch, frames, H, W = 2, 4, 12, 12
    half = torch.randint(0, 31, (batch, frames * H * W // 2), generator=g).float() / 2
    conf = torch.cat([half, 15.0 - half], dim=1)[:, torch.randperm(frames * H * W, generator=g)]
    conf = conf.reshape(batch * frames, H, W).bfloat16()
    for thr in (-0.3, 0.0, 0.25):
        mask, means = co_me_cuext.co_me_select_windows(conf.to(DEV), batch, 3, 3, thr, mode="mse", return_means=True)
        want = oracle.select_lowest_confidence(conf, batch, 3, 3, thr, mode="mse")
        flat = conf.reshape(batch, -1)
        z = (flat - flat.mean(dim=-1, keepdim=True)) / (flat.std(dim=-1, keepdim=True) + 1e-3)
        want_means = oracle.window_confidence_means(z.reshape(-1, H, W), 3, 3).float()
        assert torch.equal(means.cpu(), want_means)
        assert torch.equal(mask.cpu(), want)
        assert 0 < int(want.sum()) < want.numel()


def test_large_window_count_uses_the_global_path():
    # more than 16384 windows per batch element: the means no longer fit the per-thread registers
    conf = torch.rand(80, 45, 45, generator=torch.Generator().manual_seed(7))     # 80 * 225 = 18000 windows
    for ratio in (0.3, 0.62):
        mask = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, ratio)
        gpu_means = co_me_cuext.co_me_select_windows(conf.to(DEV), 1, 3, 3, ratio, return_means=True)[1].cpu()
        cut = torch.quantile(gpu_means.reshape(1, -1), ratio, dim=-1, keepdim=True)
        assert torch.equal(mask.cpu().reshape(1, -1), gpu_means.reshape(1, -1) < cut)


def _select_plan(conf, batch, gh, gw, threshold, start_index, mode=0):
    """come_select_plan through the C ABI -> (mask, means, offsets, prefix)."""
    from come_amd import _lib
    lib = _lib.load()
    rows, H, W = conf.shape
    M = (H // gh) * (W // gw)
    mask = torch.empty(rows, M, dtype=torch.bool, device=DEV)
    means = torch.empty(rows, M, dtype=torch.float32, device=DEV)
    offsets = torch.full((rows + 1,), -7, dtype=torch.int32, device=DEV)
    prefix = torch.full((rows, M), -7, dtype=torch.int32, device=DEV)
    _lib.check(lib.come_select_plan(conf.data_ptr(), _lib.dtype_code(conf.dtype), batch, rows // batch, H, W, gh, gw,
                                    mode, threshold, start_index, means.data_ptr(), mask.data_ptr(), offsets.data_ptr(),
                                    prefix.data_ptr(), None, 0, _lib.current_stream(conf.device)))
    return mask, means, offsets, prefix


def _plan(mask, start_index, G, tail):
    from come_amd import _lib
    lib = _lib.load()
    rows, M = mask.shape
    offsets = torch.empty(rows + 1, dtype=torch.int32, device=DEV)
    prefix = torch.empty(rows, M, dtype=torch.int32, device=DEV)
    _lib.check(lib.come_merge_plan(mask.view(torch.uint8).data_ptr(), rows, M, start_index, G, tail, offsets.data_ptr(),
                                   prefix.data_ptr(), _lib.current_stream(mask.device)))
    return offsets, prefix


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("batch,frames,H,W,gh,gw,ratio", [(1, 16, 37, 37, 3, 3, 0.5), (1, 128, 37, 28, 3, 3, 0.75),
                                                          (1, 1, 6, 6, 3, 3, 0.5), (3, 4, 12, 9, 3, 3, 0.37),
                                                          (2, 20, 37, 37, 3, 3, 0.25), (1, 80, 45, 45, 3, 3, 0.62),
                                                          (1, 7, 20, 16, 2, 4, 0.4), (2, 3, 1, 64, 1, 4, 0.5)])
def test_select_plan_is_select_then_plan(batch, frames, H, W, gh, gw, ratio, dtype):
    """One launch from the confidence to the merge plan: mask and means as come_select_windows gives them, offsets
    and prefix as come_merge_plan gives them for that mask, and against the closed form of the offsets."""
    conf = _smooth_confidence(batch * frames, H, W, seed=frames + W).to(dtype).to(DEV)
    S0 = 5
    mask, means, offsets, prefix = _select_plan(conf, batch, gh, gw, ratio, S0)
    mask_ref, means_ref = co_me_cuext.co_me_select_windows(conf, batch, gh, gw, ratio, return_means=True)
    assert torch.equal(mask, mask_ref) and torch.equal(means, means_ref)
    if gh == 3 and gw == 3 and dtype == torch.bfloat16:
        assert torch.equal(mask.cpu(), oracle.select_lowest_confidence(conf.cpu(), batch, 3, 3, ratio))
    G = gh * gw
    M = (H // gh) * (W // gw)
    tail = H * W - M * G
    offsets_ref, prefix_ref = _plan(mask, S0, G, tail)
    assert torch.equal(offsets, offsets_ref)
    assert torch.equal(prefix, prefix_ref)
    lens = S0 + tail + M * G - (G - 1) * mask.sum(dim=1)
    assert torch.equal(offsets.cpu().long(), torch.cat((torch.zeros(1, dtype=torch.long), lens.cpu().cumsum(0))))


def test_select_plan_other_modes_and_errors():
    from come_amd import _lib
    conf = torch.rand(8, 12, 12, generator=torch.Generator().manual_seed(5)).to(DEV)
    for mode, name, thr in ((1, "abs_mse", 0.5), (2, "mse", 0.0)):
        mask, _, offsets, prefix = _select_plan(conf, 2, 3, 3, thr, 0, mode=mode)
        assert torch.equal(mask, co_me_cuext.co_me_select_windows(conf, 2, 3, 3, thr, mode=name))
        o_ref, p_ref = _plan(mask, 0, 9, 0)
        assert torch.equal(offsets, o_ref) and torch.equal(prefix, p_ref)
    lib = _lib.load()
    small = torch.rand(2, 2, 2, device=DEV)                       # no full 3x3 window
    dummy = torch.empty(16, dtype=torch.int32, device=DEV)
    rc = lib.come_select_plan(small.data_ptr(), 0, 1, 2, 2, 2, 3, 3, 0, 0.5, 0, dummy.data_ptr(), dummy.data_ptr(),
                              dummy.data_ptr(), dummy.data_ptr(), None, 0, None)
    assert rc == 2 and b"no full window" in lib.come_last_error()
    # the Python operator handles that case by keeping every token
    tokens = torch.randn(2, 5 + 4, 64, device=DEV).bfloat16()
    merged, index_map, counts, cu, mask = co_me_cuext.co_me_select_merge_2d(tokens, small, 1, 5, 3, 3, 2, 2, 0.5)
    assert torch.equal(merged, tokens.reshape(-1, 64)) and cu.tolist() == [0, 9, 18] and mask.shape == (2, 0)
    assert torch.equal(index_map.cpu(), torch.arange(18, dtype=torch.int32)) and bool((counts == 1).all())


@pytest.mark.parametrize("ratio", [0.25, 0.5, 0.75])
def test_fused_select_merge_c2(ratio):
    B, S, H, W, C, S0 = 1, 16, 37, 37, 1024, 5
    g = torch.Generator().manual_seed(0)
    tokens = torch.randn(S, S0 + H * W, C, generator=g).bfloat16()
    conf = _smooth_confidence(S, H, W, seed=0)
    want_mask = oracle.select_lowest_confidence(conf, B, 3, 3, ratio)
    ref, ref_rev = oracle.token_merge_2d(tokens, S0, 3, 3, H, W, want_mask, allow_remainder=True)
    merged, index_map, counts, cu, mask = co_me_cuext.co_me_select_merge_2d(
        tokens.to(DEV), conf.to(DEV), B, S0, 3, 3, H, W, ratio)
    assert torch.equal(mask.cpu(), want_mask)
    assert index_map.dtype == torch.int32 and counts.dtype == torch.int32 and cu.dtype == torch.int32
    assert torch.equal(cu.cpu().long(), ref.offset)
    assert torch.equal(index_map.cpu().long(), ref_rev)
    assert torch.equal(counts.cpu().float(), ref.weight)
    k = {0.25: 576, 0.5: 1152, 0.75: 1728}[ratio]                  # floor(r (n-1)) + 1 of n = 2304 windows
    assert int(mask.sum()) == k and merged.shape[0] == S * (S0 + H * W) - 8 * k
    diff = (merged.float().cpu() - ref.tokens[0].float()).abs()
    assert float(diff.max()) <= 1e-2 and float(diff.mean()) <= 1e-3


def test_merger_class_round_trip():
    B, S, H, W, C, S0 = 2, 4, 12, 12, 64, 5
    merger = CoMe_2D_TokenMerger(start_idx=S0, group_h=3, group_w=3, threshold=0.5)
    conf = torch.rand(B, S * H * W).bfloat16()
    feature = torch.empty(B, S, C, H, W, device=DEV)
    ctx = merger.build_ctx(feature, confidence=conf.to(DEV))
    want = oracle.select_lowest_confidence(conf.reshape(B * S, H, W), B, 3, 3, 0.5)
    assert torch.equal(ctx[0].cpu(), want)
    tokens = torch.randn(B, S, S0 + H * W, C).bfloat16().to(DEV)
    jag, stub = merger.merge(ctx, tokens)
    back = merger.split(ctx, stub, jag)
    assert back.shape == tokens.shape
    infer = merger.build_infer_mask(ctx)
    assert infer.shape == (B, S, H, W)
    kept = ~infer.reshape(B, S, H * W)
    assert torch.equal(back[:, :, S0:][kept], tokens[:, :, S0:][kept])
    assert torch.equal(back[:, :, :S0], tokens[:, :, :S0])
    assert int(infer.sum()) == 9 * int(want.sum())
