"""Oracle: token merge / split on the CPU.  Test infrastructure only.

Restates ``func_token_merge`` / ``func_token_split``
(reference ``src/accelerate/token_merger/co_me.py:153-222, 241-254``) and the
2-D window variant ``naive_func_token_merge_2d`` / ``func_token_merge_2d``
(``src/accelerate/token_merger/co_me_2d.py:77-169, 174-211``).

Layout of one packed row block (one frame ``b``)::

    [ start_index special tokens | group 0 | group 1 | ... | tail tokens ]

where a group whose mask bit is set occupies ONE row holding the mean of its
``G`` source tokens (weight ``G``) and any other group occupies ``G`` rows that
are copies (weight 1).  ``tail`` tokens (an extension with no reference
counterpart, used for grids whose sides are not multiples of the window) are
copied behind the groups with weight 1; ``tail == 0`` is the reference layout.

The mean is taken with ``Tensor.mean`` in the token dtype, as the reference
does (``co_me.py:196-197``): for bf16 / fp16 that is an fp32 accumulation and a
single rounding.
"""

from __future__ import annotations

import torch

from .jagged import JaggedTokens


# --------------------------------------------------------------------------
# argument checks (messages follow co_me.py:108-128 / co_me_2d.py:38-72 so the
# same regular expressions match)
# --------------------------------------------------------------------------

def _check_1d(tokens, start_index, group_size, merge_mask, tail):
    if start_index < 0:
        raise ValueError(f"start_index must be >= 0, got {start_index}")
    if group_size <= 0:
        raise ValueError(f"group_size must be > 0, got {group_size}")
    if tail < 0:
        raise ValueError(f"tail must be >= 0, got {tail}")
    if merge_mask.dtype != torch.bool:
        raise ValueError(f"merge_mask must be of dtype torch.bool, got {merge_mask.dtype}")
    rows, n_tok, _ = tokens.shape
    mask_rows, n_grp = merge_mask.shape
    if mask_rows != rows:
        raise ValueError(f"merge_mask batch ({mask_rows}) must match tokens batch ({rows})")
    want = start_index + n_grp * group_size + tail
    if n_tok != want:
        raise ValueError(
            f"Expected N = start_index + M * group_size = {start_index} + {n_grp} * {group_size} = "
            f"{want}, got N = {n_tok}"
        )


def _check_2d(tokens, start_index, group_h, group_w, H, W, merge_mask, allow_remainder):
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
    rows, n_tok, _ = tokens.shape
    mask_rows, n_grp = merge_mask.shape
    if mask_rows != rows:
        raise ValueError(f"merge_mask batch ({mask_rows}) must match tokens batch ({rows})")
    if n_tok != start_index + H * W:
        raise ValueError(
            f"Expected N = start_index + H * W = {start_index} + {H * W} = "
            f"{start_index + H * W}, got N = {n_tok}"
        )
    want = (H // group_h) * (W // group_w)
    if n_grp != want:
        raise ValueError(f"Expected M = (H // group_h) * (W // group_w) = {want}, got M = {n_grp}")


# --------------------------------------------------------------------------
# 1-D merge
# --------------------------------------------------------------------------

def token_merge_1d(
    tokens: torch.Tensor,
    start_index: int,
    group_size: int,
    merge_mask: torch.Tensor,
    tail: int = 0,
) -> tuple[JaggedTokens, torch.Tensor]:
    """``tokens [B, N, C]``, ``merge_mask [B, M] bool`` ->
    ``(JaggedTokens(tokens [1,P,C], weight [P] f32, offset [B+1] i64), rev [B*N] i64)``.

    ``rev[i]`` is the packed row that source token ``i`` went to.
    Follows co_me.py:153-222 (+ ``tail`` extension).
    """
    _check_1d(tokens, start_index, group_size, merge_mask, tail)
    rows, n_tok, chans = tokens.shape
    n_grp = merge_mask.shape[1]
    G = group_size

    # rows of output each group takes, and where every frame / group starts
    rows_per_group = torch.where(merge_mask, 1, G).to(torch.int64)              # [B, M]
    frame_len = start_index + rows_per_group.sum(dim=1) + tail                   # co_me.py:177-178
    offset = torch.zeros(rows + 1, dtype=torch.int64)
    offset[1:] = torch.cumsum(frame_len, dim=0)                                  # co_me.py:180-182
    P = int(offset[-1])
    frame_base = offset[:-1]
    group_first = frame_base[:, None] + start_index + (
        torch.cumsum(rows_per_group, dim=1) - rows_per_group                      # exclusive scan, co_me.py:199-201
    )

    # destination row of every source token
    rev = torch.empty(rows, n_tok, dtype=torch.int64)
    rev[:, :start_index] = frame_base[:, None] + torch.arange(start_index)
    step = torch.arange(G)[None, None, :] * (~merge_mask)[:, :, None]            # 0,0,.. for merged groups
    rev[:, start_index:start_index + n_grp * G] = (group_first[:, :, None] + step).reshape(rows, n_grp * G)
    if tail:
        tail_first = frame_base + start_index + rows_per_group.sum(dim=1)
        rev[:, start_index + n_grp * G:] = tail_first[:, None] + torch.arange(tail)
    rev = rev.reshape(-1)

    # features: copy every token to its row, then overwrite merged rows by the group mean
    out = torch.empty(P, chans, dtype=tokens.dtype)
    out[rev] = tokens.reshape(rows * n_tok, chans)
    if n_grp > 0:
        grouped = tokens[:, start_index:start_index + n_grp * G, :].reshape(rows, n_grp, G, chans)
        out[group_first[merge_mask]] = grouped.mean(dim=2)[merge_mask]          # co_me.py:196-197, 206-207

    # weight = number of source tokens per packed row (1 or G), co_me.py:216-219
    weight = torch.zeros(P, dtype=torch.float32)
    weight.index_add_(0, rev, torch.ones(rows * n_tok, dtype=torch.float32))

    return JaggedTokens(tokens=out.unsqueeze(0), weight=weight, offset=offset), rev


def token_split(jagged: JaggedTokens, rev: torch.Tensor, bsnc_shape: tuple[int, int, int, int]) -> torch.Tensor:
    """Inverse layout step (co_me.py:241-254): row gather by ``rev`` -> ``[B*S, N, C]``."""
    B, S, N, C = bsnc_shape
    return jagged.tokens[0][rev].reshape(B * S, N, C)


# --------------------------------------------------------------------------
# 2-D window merge
# --------------------------------------------------------------------------

def window_major_permutation(H: int, W: int, group_h: int, group_w: int) -> tuple[torch.Tensor, int]:
    """Order of the ``H*W`` grid positions in the packed layout.

    Full windows first: windows in block-row-major order, positions inside a
    window row-major (co_me_2d.py:26-35).  Positions not covered by a full
    window (``y >= (H//gh)*gh`` or ``x >= (W//gw)*gw``) follow in image
    row-major order.  Returns ``(perm [H*W] int64, number_of_remainder_positions)``.
    """
    mh, mw = H // group_h, W // group_w
    ys, xs = torch.meshgrid(torch.arange(H), torch.arange(W), indexing="ij")
    covered = (ys < mh * group_h) & (xs < mw * group_w)
    # sort key: (uncovered, window row, window col, row in window, col in window) / (uncovered, y, x)
    win_key = (((ys // group_h) * mw + xs // group_w) * group_h + ys % group_h) * group_w + xs % group_w
    key = torch.where(covered, win_key, H * W + ys * W + xs)
    perm = torch.argsort(key.reshape(-1), stable=True)
    return perm, int((~covered).sum())


def token_merge_2d(
    tokens: torch.Tensor,
    start_index: int,
    group_h: int,
    group_w: int,
    H: int,
    W: int,
    merge_mask: torch.Tensor,
    allow_remainder: bool = False,
) -> tuple[JaggedTokens, torch.Tensor]:
    """2-D window merge (co_me_2d.py:77-169): tokens of every ``gh x gw`` window become
    contiguous, the 1-D merge runs on that order, and ``rev`` is reported in the
    original image row-major token order (co_me_2d.py:158-166, 204-209).
    """
    _check_2d(tokens, start_index, group_h, group_w, H, W, merge_mask, allow_remainder)
    rows, n_tok, _ = tokens.shape
    perm, tail = window_major_permutation(H, W, group_h, group_w)
    order = torch.cat([torch.arange(start_index), perm + start_index])          # packed order -> source index
    jagged, rev_packed_order = token_merge_1d(
        tokens[:, order, :], start_index, group_h * group_w, merge_mask, tail=tail
    )
    rev = torch.empty(rows, n_tok, dtype=torch.int64)
    rev[:, order] = rev_packed_order.reshape(rows, n_tok)
    return jagged, rev.reshape(-1)
