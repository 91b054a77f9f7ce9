"""1-D Co-Me token merge / split on the HIP kernels.

``func_token_merge`` / ``func_token_split`` keep the names, arguments, return values and
``ValueError`` messages of the reference (``src/accelerate/token_merger/co_me.py:108-128,
153-222, 241-254``).  There is no PyTorch fallback: both always run the HIP library.
"""

from __future__ import annotations

import inspect
from typing import Any, Callable

import torch

from ..cuda_extension.co_me import co_me_cuext
from ..interface import ITokenMerger, JaggedTokens


def _validate_token_merge_args(tokens: torch.Tensor, start_index: int, group_size: int,
                               merge_mask: torch.Tensor) -> None:
    if start_index < 0:
        raise ValueError(f"start_index must be >= 0, got {start_index}")
    if group_size <= 0:
        raise ValueError(f"group_size must be > 0, got {group_size}")
    if merge_mask.dtype != torch.bool:
        raise ValueError(f"merge_mask must be of dtype torch.bool, got {merge_mask.dtype}")
    n_rows, n_tok, _ = tokens.shape
    mask_rows, n_groups = merge_mask.shape
    if mask_rows != n_rows:
        raise ValueError(f"merge_mask batch ({mask_rows}) must match tokens batch ({n_rows})")
    expect = start_index + n_groups * group_size
    if n_tok != expect:
        raise ValueError(
            f"Expected N = start_index + M * group_size = {start_index} + {n_groups} * {group_size} = "
            f"{expect}, got N = {n_tok}"
        )


def func_token_merge(tokens: torch.Tensor, start_index: int, group_size: int,
                     merge_mask: torch.Tensor) -> tuple[JaggedTokens, torch.Tensor]:
    """``tokens [B, N, C]``, ``merge_mask [B, M] bool`` (True = replace the group of ``group_size``
    tokens by their mean) -> ``(JaggedTokens, rev_id [B*N] int64)``; ``rev_id`` maps every source
    token to its packed row."""
    _validate_token_merge_args(tokens, start_index, group_size, merge_mask)
    out_flat, offsets, rev_id, weight = co_me_cuext.co_me_token_merge_cuda(
        tokens.contiguous(), start_index, group_size, merge_mask.contiguous())
    return JaggedTokens(tokens=out_flat.unsqueeze(0), weight=weight, offset=offsets.long()), rev_id


def func_token_split(tokens: JaggedTokens, rev_id: torch.Tensor,
                     bsnc_shape: tuple[int, int, int, int]) -> torch.Tensor:
    """Inverse layout step: gather packed rows back to ``[B*S, N, C]`` with ``rev_id``."""
    B, S, N, C = bsnc_shape
    flat = tokens.tokens.squeeze(0)
    restored = co_me_cuext.co_me_token_split_cuda(flat.contiguous(), rev_id.contiguous(), C)
    return restored.reshape(B * S, N, C)


def func_token_split_pair(tokens_a: JaggedTokens, tokens_b: JaggedTokens, rev_id: torch.Tensor,
                          bsnc_shape: tuple[int, int, int, int]) -> torch.Tensor:
    """``torch.cat((func_token_split(a), func_token_split(b)), dim=-1)`` in one launch -> ``[B*S, N, 2*C]``."""
    B, S, N, C = bsnc_shape
    restored = co_me_cuext.co_me_token_split_pair_cuda(tokens_a.tokens.squeeze(0), tokens_b.tokens.squeeze(0),
                                                       rev_id.contiguous(), C)
    return restored.reshape(B * S, N, 2 * C)


def run_predictor(predictor, feature: torch.Tensor) -> torch.Tensor:
    """Confidence of ``feature [B, S, C, H, W]`` from a predictor, one scalar per patch.

    A plain callable gets the channels-last bf16 feature; the reference's predictor modules take the shape as a
    keyword as well (``forward(tokens, BPHWC)``, src/accelerate/common/confidence_predictor.py:21, 51) and are
    called the way the reference calls them (co_me.py:50, co_me_2d.py:264-267)."""
    B, S, C, H, W = feature.shape
    tokens = feature.permute(0, 1, 3, 4, 2).bfloat16()
    forward = getattr(predictor, "forward", predictor)
    try:
        wants_shape = "BPHWC" in inspect.signature(forward).parameters
    except (TypeError, ValueError):
        wants_shape = False
    confidence = predictor(tokens, BPHWC=(B, S, H, W, C)) if wants_shape else predictor(tokens)
    if confidence.numel() != B * S * H * W:
        raise ValueError(f"the predictor must return one confidence per patch ({B * S * H * W}), "
                         f"got a tensor of shape {tuple(confidence.shape)}")
    return confidence


class CoMe_TokenMerger(ITokenMerger):
    """Groups of ``group_size`` consecutive tokens (reference ``CoMe_TokenMerger``, co_me.py:20-105).

    The confidence predictor is outside this package: pass a callable
    ``predictor(feature [B,S,H,W,C] bf16) -> confidence [B, S*H*W]`` (the reference's predictor modules work
    as they are) or hand the confidence to ``build_ctx`` directly.  ``conf_mode`` uses the reference's names.
    """

    def __init__(self, start_idx: int, group_size: int, threshold: float,
                 predictor: Callable[[torch.Tensor], torch.Tensor] | None = None,
                 conf_mode: str = "pairwise-rank"):
        self.start_idx = start_idx
        self.group_size = group_size
        self.threshold = threshold
        self.predictor = predictor
        self.conf_mode = conf_mode

    def build_ctx(self, feature: torch.Tensor, confidence: torch.Tensor | None = None) -> Any:
        B, S, C, H, W = feature.shape
        if (H * W) % self.group_size != 0:
            raise ValueError(f"H * W ({H * W}) must be divisible by group_size ({self.group_size})")
        if confidence is None:
            if self.predictor is None:
                raise ValueError("build_ctx needs a confidence tensor or a predictor")
            confidence = run_predictor(self.predictor, feature)
        if self.conf_mode == "pairwise-rank" and not (0.0 <= self.threshold <= 1.0):
            raise ValueError(f"Ranking mode requires threshold in [0, 1], got {self.threshold}")
        # groups of G consecutive tokens are 1 x G windows of a 1 x (H*W) grid.  Scope of the statistics as in the
        # reference: the ranking takes its quantile over the last dimension of [B*S, M], i.e. per frame
        # (co_me.py:65-70), the normalised score is normalised over the whole batch element (co_me.py:54-58)
        conf = confidence.reshape(B * S, 1, H * W)
        batch = B if self.conf_mode == "mse" else B * S
        mask = co_me_cuext.co_me_select_windows(conf, batch, 1, self.group_size, self.threshold, self.conf_mode)
        return mask, (B, S, C, H, W)

    def merge(self, ctx, tokens: torch.Tensor, stub: Any | None = None, *, start_index: int | None = None):
        mask, _ = ctx
        si = self.start_idx if start_index is None else start_index
        merged, rev_id = func_token_merge(tokens.flatten(0, 1), si, self.group_size, mask)
        return merged, (rev_id, tokens.shape)

    def split(self, ctx, stub: Any, tokens: JaggedTokens) -> torch.Tensor:
        rev_id, shape_bsnc = stub
        B, S, N, C = shape_bsnc
        return func_token_split(tokens, rev_id, shape_bsnc).view(B, S, N, C)

    def split_pair(self, ctx, stub: Any, tokens_a: JaggedTokens, tokens_b: JaggedTokens) -> torch.Tensor:
        """``torch.cat((split(a), split(b)), dim=-1)`` in one launch -> ``[B, S, N, 2*C]``."""
        rev_id, shape_bsnc = stub
        B, S, N, C = shape_bsnc
        return func_token_split_pair(tokens_a, tokens_b, rev_id, shape_bsnc).view(B, S, N, 2 * C)

    def build_infer_mask(self, ctx) -> torch.Tensor:
        mask, (B, S, _, H, W) = ctx
        return mask.unsqueeze(-1).repeat(1, 1, self.group_size).flatten(-2, -1).reshape(B, S, H, W)
