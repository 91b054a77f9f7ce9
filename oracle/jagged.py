"""Packed ("jagged") token container of the oracle.  Test infrastructure only.

Same three fields as the reference's ``ITokenMerger.JaggedTokens``
(``src/interface/token_merger.py:12-21``): ``tokens [1, P, C]``,
``weight [P]`` (how many source tokens each packed row stands for) and
``offset [n_seg + 1]`` (segment boundaries, int64), and its two suffix operators
(``:23-100``), restated segment by segment and pinned by the reference's three known-answer
cases (``tests/golden/suffix.json``) and the round trip.
"""

from dataclasses import dataclass

import torch


@dataclass
class JaggedTokens:
    tokens: torch.Tensor
    weight: torch.Tensor
    offset: torch.Tensor


def add_suffix(jagged: JaggedTokens, suffix: torch.Tensor) -> JaggedTokens:
    """Appends ``suffix[m]`` (``[T, C]``, weight 1) to segment ``m`` (``src/interface/token_merger.py:23-58``)."""
    M = jagged.offset.shape[0] - 1
    if suffix.shape[0] != M:
        raise ValueError(f"suffix batch dim ({suffix.shape[0]}) must match segment count ({M})")
    T = suffix.shape[1]
    bounds = jagged.offset.tolist()
    rows, weights, offsets = [], [], [0]
    for m in range(M):
        rows += [jagged.tokens[0, bounds[m]:bounds[m + 1]], suffix[m].to(jagged.tokens.dtype)]
        weights += [jagged.weight[bounds[m]:bounds[m + 1]], torch.ones(T, dtype=jagged.weight.dtype)]
        offsets.append(offsets[-1] + bounds[m + 1] - bounds[m] + T)
    C = jagged.tokens.shape[2]
    tokens = torch.cat(rows) if rows else jagged.tokens.new_zeros(0, C)
    weight = torch.cat(weights) if weights else jagged.weight.new_zeros(0)
    return JaggedTokens(tokens=tokens.unsqueeze(0), weight=weight, offset=torch.tensor(offsets, dtype=jagged.offset.dtype))


def split_suffix(jagged: JaggedTokens, count: int) -> tuple[JaggedTokens, torch.Tensor]:
    """Strips the last ``count`` rows of every segment (``src/interface/token_merger.py:60-100``);
    returns ``(stripped, suffix [M, count, C])``."""
    M = jagged.offset.shape[0] - 1
    P, C = jagged.tokens.shape[1], jagged.tokens.shape[2]
    if P - M * count < 0:
        raise ValueError(f"Cannot strip {count} tokens from each of {M} segments (total tokens = {P})")
    bounds = jagged.offset.tolist()
    if any(bounds[m + 1] - bounds[m] < count for m in range(M)):
        raise ValueError(f"count={count} exceeds the length of at least one segment")
    rows, weights, tails, offsets = [], [], [], [0]
    for m in range(M):
        rows.append(jagged.tokens[0, bounds[m]:bounds[m + 1] - count])
        weights.append(jagged.weight[bounds[m]:bounds[m + 1] - count])
        tails.append(jagged.tokens[0, bounds[m + 1] - count:bounds[m + 1]])
        offsets.append(offsets[-1] + bounds[m + 1] - bounds[m] - count)
    tokens = torch.cat(rows) if rows else jagged.tokens.new_zeros(0, C)
    weight = torch.cat(weights) if weights else jagged.weight.new_zeros(0)
    suffix = torch.stack(tails) if tails else jagged.tokens.new_zeros(0, count, C)
    stripped = JaggedTokens(tokens=tokens.unsqueeze(0), weight=weight, offset=torch.tensor(offsets, dtype=jagged.offset.dtype))
    return stripped, suffix
