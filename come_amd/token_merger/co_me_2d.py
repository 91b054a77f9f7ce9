"""2-D (window) Co-Me token merge on the HIP kernels.

Mirrors ``src/accelerate/token_merger/co_me_2d.py`` of the reference: argument checks and
messages (``:38-72``), ``func_token_merge_2d`` / ``naive_func_token_merge_2d`` (``:77-211``) and
the merger class (``:214-352``).  Differences, all additive:

* the kernel reads windows straight from the image row-major token order, so there is no
  permuted copy of the tokens and no index remapping pass;
* ``allow_remainder=True`` accepts grids whose sides are not multiples of the window: the
  positions outside the full windows are kept, behind the windows, in image row-major order.
  The default rejects such grids exactly as the reference does;
* the confidence predictor is not part of this package (a callable or the confidence itself is
  passed in) and window reduction + selection run in one HIP kernel.
"""

from __future__ import annotations

from typing import Any, Callable

import torch

from ..cuda_extension.co_me import co_me_cuext
from ..interface import ITokenMerger, JaggedTokens
from .co_me import func_token_split, func_token_split_pair, run_predictor


def _validate_token_merge_2d_args(tokens, start_index, group_h, group_w, H, W, merge_mask,
                                  allow_remainder: bool = False) -> None:
    if start_index < 0:
        raise ValueError(f"start_index must be >= 0, got {start_index}")
    if group_h <= 0 or group_w <= 0:
        raise ValueError(f"group_h and group_w must be > 0, got ({group_h}, {group_w})")
    if not allow_remainder:
        if H % group_h != 0:
            raise ValueError(f"H ({H}) must be divisible by group_h ({group_h})")
        if W % group_w != 0:
            raise ValueError(f"W ({W}) must be divisible by group_w ({group_w})")
    if merge_mask.dtype != torch.bool:
        raise ValueError(f"merge_mask must be of dtype torch.bool, got {merge_mask.dtype}")
    n_rows, n_tok, _ = tokens.shape
    mask_rows, n_groups = merge_mask.shape
    if mask_rows != n_rows:
        raise ValueError(f"merge_mask batch ({mask_rows}) must match tokens batch ({n_rows})")
    if n_tok != start_index + H * W:
        raise ValueError(
            f"Expected N = start_index + H * W = {start_index} + {H * W} = {start_index + H * W}, got N = {n_tok}"
        )
    expect = (H // group_h) * (W // group_w)
    if n_groups != expect:
        raise ValueError(f"Expected M = (H // group_h) * (W // group_w) = {expect}, got M = {n_groups}")


def func_token_merge_2d(tokens: torch.Tensor, start_index: int, group_h: int, group_w: int, H: int, W: int,
                        merge_mask: torch.Tensor, allow_remainder: bool = False) -> tuple[JaggedTokens, torch.Tensor]:
    """``tokens [B, start_index + H*W, C]``, ``merge_mask [B, M] bool`` -> ``(JaggedTokens, rev_id [B*N] int64)``
    with ``rev_id`` in the original image row-major token order."""
    _validate_token_merge_2d_args(tokens, start_index, group_h, group_w, H, W, merge_mask, allow_remainder)
    out_flat, offsets, rev_id, weight = co_me_cuext.co_me_token_merge_2d_cuda(
        tokens, start_index, group_h, group_w, H, W, merge_mask)
    return JaggedTokens(tokens=out_flat.unsqueeze(0), weight=weight, offset=offsets.long()), rev_id


# the reference keeps a pure-PyTorch variant under this name; here both names run the same kernel
naive_func_token_merge_2d = func_token_merge_2d


class CoMe_2D_TokenMerger(ITokenMerger):
    """``group_h x group_w`` window merger (reference ``_CoMe_2D_Base`` / ``CoMe_2D_TokenMerger``)."""

    def __init__(self, start_idx: int, group_h: int, group_w: int, threshold: float,
                 predictor: Callable[[torch.Tensor], torch.Tensor] | None = None,
                 conf_mode: str = "pairwise-rank", allow_remainder: bool = False):
        self.start_idx = start_idx
        self.group_h = group_h
        self.group_w = group_w
        self.threshold = threshold
        self.predictor = predictor
        self.conf_mode = conf_mode
        self.allow_remainder = allow_remainder

    def build_ctx(self, feature: torch.Tensor, confidence: torch.Tensor | None = None) -> Any:
        """``feature [B, S, C, H, W]`` (only its shape is used when ``confidence`` is given);
        ``confidence`` holds one scalar per patch, any shape with ``B*S*H*W`` elements."""
        B, S, C, H, W = feature.shape
        if not self.allow_remainder:
            if H % self.group_h != 0:
                raise ValueError(f"H ({H}) must be divisible by group_h ({self.group_h})")
            if W % self.group_w != 0:
                raise ValueError(f"W ({W}) must be divisible by group_w ({self.group_w})")
        if confidence is None:
            if self.predictor is None:
                raise ValueError("build_ctx needs a confidence tensor or a predictor")
            confidence = run_predictor(self.predictor, feature)
        if self.conf_mode == "pairwise-rank" and not (0.0 <= self.threshold <= 1.0):
            raise ValueError(f"Ranking mode requires threshold in [0, 1], got {self.threshold}")
        mask = co_me_cuext.co_me_select_windows(confidence.reshape(B * S, H, W), B, self.group_h, self.group_w,
                                                self.threshold, self.conf_mode)
        return mask, (B, S, C, H, W)

    def merge(self, ctx: Any, tokens: torch.Tensor, stub: Any | None = None, *, start_index: int | None = None):
        mask, (B, S, C, H, W) = ctx
        si = self.start_idx if start_index is None else start_index
        merged, rev_id = func_token_merge_2d(tokens.flatten(0, 1), si, self.group_h, self.group_w, H, W, mask,
                                             allow_remainder=self.allow_remainder)
        return merged, (rev_id, tokens.shape)

    def split(self, ctx: Any, stub: Any, tokens: JaggedTokens) -> torch.Tensor:
        rev_id, shape_bsnc = stub
        B, S, N, C = shape_bsnc
        return func_token_split(tokens, rev_id, shape_bsnc).view(B, S, N, C)

    def split_pair(self, ctx: Any, stub: Any, tokens_a: JaggedTokens, tokens_b: JaggedTokens) -> torch.Tensor:
        """``torch.cat((split(a), split(b)), dim=-1)`` in one launch -> ``[B, S, N, 2*C]``."""
        rev_id, shape_bsnc = stub
        B, S, N, C = shape_bsnc
        return func_token_split_pair(tokens_a, tokens_b, rev_id, shape_bsnc).view(B, S, N, 2 * C)

    def build_infer_mask(self, ctx: Any) -> torch.Tensor:
        """``[B, S, H, W] bool``: True where the patch was merged (positions outside full windows: False)."""
        mask, (B, S, _, H, W) = ctx
        mh, mw = H // self.group_h, W // self.group_w
        full = mask.reshape(B * S, mh, 1, mw, 1).expand(-1, -1, self.group_h, -1, self.group_w)
        full = full.reshape(B * S, mh * self.group_h, mw * self.group_w)
        out = torch.zeros(B * S, H, W, dtype=torch.bool, device=mask.device)
        out[:, : mh * self.group_h, : mw * self.group_w] = full
        return out.reshape(B, S, H, W)


Naive_CoMe_2D_TokenMerger = CoMe_2D_TokenMerger
