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


def test_other_modes():
    conf = torch.rand(4, 6, 6)
    m = oracle.window_confidence_means(conf, 3, 3)
    assert torch.equal(oracle.select_lowest_confidence(conf, 1, 3, 3, 0.45, mode="abs_mse"), m < 0.45)
    z = (conf.reshape(1, -1) - conf.mean()) / (conf.reshape(-1).std() + 1e-3)
    want = oracle.window_confidence_means(z.reshape(4, 6, 6), 3, 3) < 0.1
    assert torch.equal(oracle.select_lowest_confidence(conf, 1, 3, 3, 0.1, mode="mse"), want)
    with pytest.raises(ValueError, match="threshold in"):
        oracle.select_lowest_confidence(conf, 1, 3, 3, 1.5)
