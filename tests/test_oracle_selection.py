"""Pins for the window-confidence reduction and lowest-confidence selection
oracle (no reference test covers this function; see oracle/selection.py)."""

import math

import numpy as np
import pytest
import torch

import oracle


def _loops_means(conf, gh, gw):
    F, H, W = conf.shape
    mh, mw = H // gh, W // gw
    out = np.zeros((F, mh * mw))
    for f in range(F):
        for wy in range(mh):
            for wx in range(mw):
                acc = 0.0
                for dy in range(gh):
                    for dx in range(gw):
                        acc += float(conf[f, wy * gh + dy, wx * gw + dx])
                out[f, wy * mw + wx] = acc / (gh * gw)
    return out


@pytest.mark.parametrize("F,H,W,gh,gw", [(2, 6, 6, 3, 3), (3, 7, 8, 3, 3), (1, 37, 37, 3, 3), (2, 4, 6, 2, 3)])
def test_window_means_vs_loops(F, H, W, gh, gw):
    conf = torch.rand(F, H, W, dtype=torch.float64)
    got = oracle.window_confidence_means(conf, gh, gw).numpy()
    np.testing.assert_allclose(got, _loops_means(conf.numpy(), gh, gw), rtol=1e-13, atol=0)


def test_window_means_bf16_single_rounding():
    conf = torch.rand(4, 9, 12).bfloat16()
    got = oracle.window_confidence_means(conf, 3, 3)
    assert got.dtype == torch.bfloat16
    want = torch.from_numpy(_loops_means(conf.float().numpy(), 3, 3)).bfloat16()   # fp64 mean, one rounding
    assert torch.equal(got, want)


@pytest.mark.parametrize("n,ratio", [(8, 0.5), (2304, 0.25), (2304, 0.5), (2304, 0.75), (4608, 0.6), (13824, 0.75),
                                     (100, 0.0), (100, 1.0), (1, 0.3), (17, 0.37)])
def test_quantile_restatement_matches_torch_and_numpy(n, ratio):
    x = torch.rand(n)
    t = float(torch.quantile(x, ratio))
    mine = float(oracle.quantile_threshold(x.numpy(), ratio))
    assert mine == t                                              # bit-for-bit with the library call
    ref64 = float(np.quantile(x.double().numpy(), float(np.float32(ratio))))
    assert abs(mine - ref64) <= 2e-7


@pytest.mark.parametrize("n,ratio", [(8, 0.5), (2304, 0.25), (2304, 0.5), (2304, 0.75), (4608, 0.6)])
def test_selected_count_closed_form_distinct_values(n, ratio):
    # distinct values, r(n-1) not an integer  ->  exactly floor(r(n-1)) + 1 windows lie below the threshold
    vals = torch.randperm(n).float().reshape(1, n // 4, 2, 2)      # 2x2 windows of one value each
    conf = vals.repeat_interleave(2, dim=2).repeat_interleave(2, dim=3).reshape(n // 4, 4, 4)
    rank = float(np.float32(ratio) * np.float32(n - 1))
    assert rank != math.floor(rank)
    mask = oracle.select_lowest_confidence(conf, 1, 2, 2, ratio)
    assert mask.shape == (n // 4, 4)
    assert int(mask.sum()) == math.floor(rank) + 1
    means = oracle.window_confidence_means(conf, 2, 2).reshape(-1)
    chosen = means[mask.reshape(-1)]
    assert float(chosen.max()) < float(means[~mask.reshape(-1)].min())   # really the lowest ones


def test_selection_is_joint_over_frames_and_strict():
    # two frames; all low values sit in frame 0 -> every window of frame 0 merges, none of frame 1
    conf = torch.cat([torch.zeros(1, 6, 6), torch.ones(1, 6, 6)])
    conf[0] += torch.arange(36).reshape(6, 6) * 1e-4
    conf[1] += torch.arange(36).reshape(6, 6) * 1e-4
    mask = oracle.select_lowest_confidence(conf, 1, 3, 3, 0.5)
    assert mask.tolist() == [[True] * 4, [False] * 4]
    # as two separate batch elements the same maps merge half of each frame
    mask2 = oracle.select_lowest_confidence(conf, 2, 3, 3, 0.5)
    assert mask2.sum(1).tolist() == [2, 2]
    # ties at the threshold are NOT merged (strict <)
    tie = torch.ones(1, 6, 6)
    assert int(oracle.select_lowest_confidence(tie, 1, 3, 3, 0.5).sum()) == 0


def test_bf16_path_matches_manual_composition():
    conf = torch.rand(8, 37, 37).bfloat16()
    mask = oracle.select_lowest_confidence(conf, 2, 3, 3, 0.5)
    means = oracle.window_confidence_means(conf, 3, 3).float().reshape(2, -1)
    for b in range(2):
        cut = oracle.quantile_threshold(means[b].numpy(), 0.5)
        assert torch.equal(mask.reshape(2, -1)[b], means[b] < float(cut))


def test_absolute_mode_and_validation():
    conf = torch.rand(4, 6, 6)
    m = oracle.window_confidence_means(conf, 3, 3)
    assert torch.equal(oracle.select_lowest_confidence(conf, 1, 3, 3, 0.45, mode="abs_mse"), m < 0.45)
    with pytest.raises(ValueError, match="threshold in"):
        oracle.select_lowest_confidence(conf, 1, 3, 3, 1.5)
    with pytest.raises(ValueError, match="unknown confidence mode"):
        oracle.select_lowest_confidence(conf, 1, 3, 3, 0.5, mode="nope")


# ---- normalised-score ("mse") branch: pinned by arithmetic that does not repeat the oracle's formula ----

def _hand_case():
    """One batch element holding the values 0, 1, 2, 3 (1 x 1 windows of a 2 x 2 grid).
    By hand: mean 1.5; squared deviations 2.25, 0.25, 0.25, 2.25, sum 5; unbiased variance 5 / 3,
    standard deviation 1.2909944...; denominator 1.2919944...; z = (-1.5, -0.5, 0.5, 1.5) / 1.2919944
    = (-1.1609958, -0.3869986, 0.3869986, 1.1609958)."""
    return torch.tensor([[[0.0, 1.0], [2.0, 3.0]]])


@pytest.mark.parametrize("select", ["2d", "1d"])
def test_normalised_score_hand_computed_case(select):
    conf = _hand_case()

    def mask_at(thr):
        if select == "2d":
            return oracle.select_lowest_confidence(conf, 1, 1, 1, thr, mode="mse").reshape(-1).tolist()
        return oracle.select_groups_1d(conf.reshape(1, 4), 1, 1, 1, thr, mode="mse").reshape(-1).tolist()

    z = [-1.1609958, -0.3869986, 0.3869986, 1.1609958]            # hand-computed, see _hand_case
    for thr in (-1.5, -1.0, -0.5, -0.3, 0.0, 0.4, 1.0, 1.2):
        assert mask_at(thr) == [v < thr for v in z]
    # a biased deviation (divisor n: 1.1180340 + 1e-3) would give z0 = -1.3404 and select window 0 at -1.25
    assert mask_at(-1.25) == [False, False, False, False]
    # without the "+ 1e-3" z0 would be -1.5 / 1.2909944 = -1.1618950: -1.1615 separates the two
    assert mask_at(-1.1615) == [False, False, False, False]
    assert mask_at(-1.1605) == [True, False, False, False]


@pytest.mark.parametrize("batch,frames,H,W,gh,gw", [(2, 2, 6, 6, 3, 3), (1, 3, 7, 8, 3, 3), (3, 1, 4, 6, 2, 3)])
def test_normalised_score_vs_fp64_loops(batch, frames, H, W, gh, gw):
    from bruteforce import zscore_window_means_loops

    conf = torch.rand(batch * frames, H, W, generator=torch.Generator().manual_seed(H * W + batch)) * 3 + 1
    z_means = zscore_window_means_loops(conf.double().numpy(), batch, gh, gw)
    # thresholds in the gaps of the brute-force values, so that fp32 rounding cannot move a window across
    flat = np.sort(z_means.reshape(-1))
    gaps = [(flat[i] + flat[i + 1]) / 2 for i in range(len(flat) - 1) if flat[i + 1] - flat[i] > 1e-4]
    assert len(gaps) >= 3
    for thr in gaps[:: max(1, len(gaps) // 5)]:
        got = oracle.select_lowest_confidence(conf, batch, gh, gw, float(thr), mode="mse")
        assert got.numpy().tolist() == (z_means < thr).tolist()
    # the statistics are per batch element: scaling one element's confidence must not change the others' masks
    if batch > 1:
        thr = float(gaps[len(gaps) // 2])
        base = oracle.select_lowest_confidence(conf, batch, gh, gw, thr, mode="mse")
        conf2 = conf.clone()
        conf2[:frames] = conf2[:frames] * 7 + 3                     # z-scores are invariant to an affine map ...
        again = oracle.select_lowest_confidence(conf2, batch, gh, gw, thr, mode="mse")
        assert torch.equal(again[frames:], base[frames:])           # ... and other elements never see it
        assert (again[:frames] != base[:frames]).float().mean() < 0.1


def test_1d_groups_scopes():
    """1-D merger: ranking is per frame, normalisation per batch element (reference co_me.py:54-58, 65-70)."""
    from bruteforce import zscore_window_means_loops

    B, S, HW, G = 2, 3, 16, 4
    conf = torch.rand(B, S * HW, generator=torch.Generator().manual_seed(3))
    conf[:, :HW] += 2.0                                              # frame 0 of every element is much more confident
    rank = oracle.select_groups_1d(conf, B, S, G, 0.5, mode="pairwise-rank")
    assert rank.shape == (B * S, HW // G)
    assert rank.sum(dim=1).tolist() == [2] * (B * S)                 # per frame: half of every frame's 4 groups
    means = conf.reshape(B * S, HW // G, G).mean(-1)
    for f in range(B * S):
        assert torch.equal(rank[f], means[f] < float(oracle.quantile_threshold(means[f].numpy(), 0.5)))
    # normalised score against the loops: groups of G consecutive scores are 1 x G windows of a 1 x HW grid,
    # statistics over all S frames of the element
    z_means = zscore_window_means_loops(conf.reshape(B * S, 1, HW).double().numpy(), B, 1, G)
    for thr in (-0.8, -0.2, 0.3):
        assert float(np.abs(z_means - thr).min()) > 1e-4
        got = oracle.select_groups_1d(conf, B, S, G, thr, mode="mse")
        assert got.numpy().tolist() == (z_means < thr).tolist()
    # per-frame statistics would give a different answer on this data (frame 0 is offset by +2)
    per_frame = zscore_window_means_loops(conf.reshape(B * S, 1, HW).double().numpy(), B * S, 1, G)
    assert ((per_frame < -0.2) != (z_means < -0.2)).any()
    absm = oracle.select_groups_1d(conf, B, S, G, 0.6, mode="abs_mse")
    assert torch.equal(absm, means < 0.6)
