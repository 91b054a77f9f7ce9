"""Oracle: window confidence reduction and lowest-confidence selection.
Test infrastructure only.

Restates the ``Ranking`` branch of ``_CoMe_2D_Base.build_ctx``
(reference ``src/accelerate/token_merger/co_me_2d.py:253-313``), plus the two
other modes of the same function (``Absolute_Score``, ``Normalized_Score``).

PARITY UNPINNED by the reference's own tests (no test there calls
``build_ctx``).  What pins it in this repository: the composition below uses
the very library calls the reference makes (``Tensor.mean``,
``torch.quantile``, ``<``); ``quantile_threshold`` is an independent sort-based
restatement of ``torch.quantile`` checked against it and against
``numpy.quantile``; and for distinct values the number of selected windows has
the closed form ``floor(r (n-1)) + 1`` (``r (n-1)`` not an integer).  The
normalised-score branch is pinned by a hand-computed case (values 0..3: mean
1.5, unbiased standard deviation sqrt(5/3)) whose thresholds separate it from
a biased deviation and from a missing ``+ 1e-3``, and by an fp64 loop brute
force (``tests/bruteforce.py``).  ``select_groups_1d`` restates the 1-D
merger's ``build_ctx`` (``src/accelerate/token_merger/co_me.py:47-73``) and is
pinned the same way plus by its per-frame / per-batch-element scope.
"""

from __future__ import annotations

import math

import numpy as np
import torch


def window_confidence_means(conf: torch.Tensor, group_h: int, group_w: int) -> torch.Tensor:
    """``conf [F, H, W]`` (bf16 or fp32) -> per-window mean ``[F, M]`` in ``conf.dtype``.

    Windows in block-row-major order, only full windows (co_me_2d.py:270-272, 291;
    positions outside the full windows never take part).  ``Tensor.mean`` on bf16 is
    an fp32 accumulation followed by one rounding to bf16.
    """
    F, H, W = conf.shape
    mh, mw = H // group_h, W // group_w
    core = conf[:, : mh * group_h, : mw * group_w]
    blocks = core.reshape(F, mh, group_h, mw, group_w).permute(0, 1, 3, 2, 4)
    blocks = blocks.reshape(F, mh * mw, group_h * group_w)
    return blocks.mean(dim=-1)


def quantile_threshold(values: np.ndarray, ratio: float) -> np.float32:
    """Sort-based restatement of ``torch.quantile(x.float(), ratio)`` (linear interpolation).

    ``rank = float32(ratio) * (n - 1)`` evaluated in fp32, neighbours
    ``a = sorted[floor(rank)]``, ``b = sorted[ceil(rank)]``, ``w = rank - floor(rank)``
    and ``a + w (b - a)`` for ``w < 0.5`` else ``b - (b - a)(1 - w)``, all in fp32.
    """
    x = np.sort(np.asarray(values, dtype=np.float32))
    n = x.shape[0]
    rank = np.float32(ratio) * np.float32(n - 1)
    lo = int(math.floor(float(rank)))
    hi = int(math.ceil(float(rank)))
    w = np.float32(rank - np.float32(lo))
    a, b = x[lo], x[hi]
    if w < np.float32(0.5):
        return np.float32(a + w * np.float32(b - a))
    return np.float32(b - np.float32(b - a) * np.float32(np.float32(1.0) - w))


def select_lowest_confidence(
    conf: torch.Tensor,
    batch: int,
    group_h: int,
    group_w: int,
    threshold: float,
    mode: str = "pairwise-rank",
) -> torch.Tensor:
    """``conf [B*S, H, W]`` -> ``mask [B*S, M] bool`` (True = merge this window).

    ``mode`` uses the reference's names (co_me_2d.py:218-221):
      * ``"pairwise-rank"`` (Ranking, the shipped mode): per batch element, over all
        of its ``S*M`` windows jointly, ``mask = mean < quantile(mean.float(), threshold)``
        (co_me_2d.py:285-295).
      * ``"abs_mse"`` (Absolute_Score): ``mask = mean < threshold`` (co_me_2d.py:297-298).
      * ``"mse"`` (Normalized_Score): z-score of the per-position confidence over the
        batch element (``std + 1e-3``), window mean of that, ``< threshold``
        (co_me_2d.py:275-283).
    """
    F, H, W = conf.shape
    if F % batch != 0:
        raise ValueError(f"conf rows ({F}) must be a multiple of batch ({batch})")
    if mode == "pairwise-rank":
        if not (0.0 <= threshold <= 1.0):
            raise ValueError(f"Ranking mode requires threshold in [0, 1], got {threshold}")
        means = window_confidence_means(conf, group_h, group_w)
        per_batch = means.reshape(batch, -1)
        cut = torch.quantile(per_batch.float(), threshold, dim=-1, keepdim=True)
        return (per_batch < cut).reshape(F, -1)
    if mode == "abs_mse":
        return window_confidence_means(conf, group_h, group_w) < threshold
    if mode == "mse":
        flat = conf.reshape(batch, -1)
        z = (flat - flat.mean(dim=-1, keepdim=True)) / (flat.std(dim=-1, keepdim=True) + 1e-3)
        return window_confidence_means(z.reshape(F, H, W), group_h, group_w) < threshold
    raise ValueError(f"unknown confidence mode {mode!r}")


def select_groups_1d(
    confidence: torch.Tensor,
    batch: int,
    frames: int,
    group_size: int,
    threshold: float,
    mode: str = "pairwise-rank",
) -> torch.Tensor:
    """1-D merger: ``confidence [B, S*H*W]`` -> ``mask [B*S, H*W // G] bool``.

    Restates ``CoMe_TokenMerger.build_ctx`` (reference
    ``src/accelerate/token_merger/co_me.py:47-73``).  Scope of each mode there:
      * ``"mse"``: z-score over the whole batch element (``[B, -1]``, ``:54-58``),
        then the mean of each group of ``G`` consecutive scores;
      * ``"pairwise-rank"``: the quantile is taken over the last dimension of
        ``[B*S, M]``, i.e. per frame (``:65-70``), not jointly as in the 2-D merger;
      * ``"abs_mse"``: group mean ``< threshold`` (``:72-74``).
    """
    per_frame = confidence.numel() // (batch * frames)
    if per_frame % group_size != 0:
        raise ValueError(f"H * W ({per_frame}) must be divisible by group_size ({group_size})")
    groups = per_frame // group_size
    if mode == "mse":
        flat = confidence.reshape(batch, -1)
        z = (flat - flat.mean(dim=-1, keepdim=True)) / (flat.std(dim=-1, keepdim=True) + 1e-3)
        return z.reshape(batch * frames, groups, group_size).mean(dim=-1) < threshold
    means = confidence.reshape(batch * frames, groups, group_size).mean(dim=-1)
    if mode == "pairwise-rank":
        if not (0.0 <= threshold <= 1.0):
            raise ValueError(f"Ranking mode requires threshold in [0, 1], got {threshold}")
        cut = torch.quantile(means.float(), threshold, dim=-1, keepdim=True)
        return means < cut
    if mode == "abs_mse":
        return means < threshold
    raise ValueError(f"unknown confidence mode {mode!r}")
